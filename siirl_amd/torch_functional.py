"""Log-prob / entropy from logits and masked reductions, with the reference's Python signatures.

Mirror of ``siirl/utils/model_utils/torch_functional.py:41-168`` of the reference: same names, same
argument meaning.  The arithmetic runs in ``libsiirl_hip.so``; tensors must live on the GPU.

Differences a caller can observe, all deliberate:

* results for 16-bit logits are fp32 (what the reference returns on its flash-attn dispatch,
  ``torch_functional.py:73-79,85-90``); accumulation is always fp32; float64 logits are computed in fp32
  (rounded once on entry) and the results returned as float64;
* ``logprobs_from_logits`` also computes the entropy in the same pass over the row and keeps it with the
  returned log-probs, so that the ``entropy_from_logits(logits)`` call that the actor issues next on the same
  tensor (``siirl/engine/actor/dp_actor.py:179-195,254-260``) costs no second pass and both gradients are written
  by one backward kernel.  ``set_pairing(False)`` turns this off;
* a label of ``-101`` (``siirl_amd.padding.LABEL_SKIP_ROW``, set by ``unpad_ids_and_labels(..., response_length=L)``
  on the packed tokens outside the response window) makes both passes skip the row: log-prob and entropy 0, zero
  gradient, the logits of the row are never read (the single-launch step, ``fused_actor_step``, does the same);
* opt-in (``set_skip_zero_rows(True)``): the backward writes zeros, without reading the row, where both upstream
  gradients of a row are zero; a NaN or Inf in a padded row's logits then does not reach ``dlogits`` as it would
  through the reference's autograd, so the default leaves it off.
"""

from __future__ import annotations

import threading
import weakref

import torch

from . import ops  # noqa: F401  (loads torch.ops.siirl_hip.*)

_OPS = torch.ops.siirl_hip
_fwd = _OPS.logprob_entropy_fwd
_bwd = _OPS.logprob_entropy_bwd
_bwd_ = _OPS.logprob_entropy_bwd_
_lpe = _OPS.logprob_entropy.default

_SKIP_ZERO_ROWS = False


def set_skip_zero_rows(flag: bool) -> None:
    """``True``: the backward writes zeros, without reading the row, where both upstream gradients are zero
    (padding rows).  Identical results for finite logits; a NaN or Inf in such a row then no longer reaches
    ``dlogits`` as it does through the reference's autograd (``0 * NaN``), which is why it is off by default."""
    global _SKIP_ZERO_ROWS
    _SKIP_ZERO_ROWS = bool(flag)


class _LogprobEntropy(torch.autograd.Function):
    """(logits, labels) -> (logprob, entropy) over the plain operators, which are opaque to Dynamo and have fake
    kernels: the form a ``torch.compile(fullgraph=True)`` region can hold (``logprob_entropy_traceable``).  Everything
    else uses the C++ node ``logprob_entropy``."""

    @staticmethod
    def forward(ctx, logits, labels, inv_temperature, want_entropy, inplace_backward):
        lp, ent, lse, ex = _fwd(logits, labels, inv_temperature, want_entropy)
        ctx.save_for_backward(logits, labels if labels is not None else lse.new_empty(0), lse, ex)
        ctx.has_labels = labels is not None
        ctx.want_entropy = want_entropy
        ctx.inv_temperature = inv_temperature
        ctx.inplace = inplace_backward
        ctx.set_materialize_grads(False)
        if labels is None:
            ctx.mark_non_differentiable(lp)
        if not want_entropy:
            ctx.mark_non_differentiable(ent)
        return lp, ent

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        logits, labels, lse, ex = ctx.saved_tensors
        if not ctx.has_labels:
            labels, g_lp = None, None
        if not ctx.want_entropy:
            g_ent = None
        if g_lp is None and g_ent is None:
            return None, None, None, None, None
        args = (logits, labels, ctx.inv_temperature, lse,  # (labels also mark the rows the forward skipped)
                ex if g_ent is not None else None, g_lp, g_ent, _SKIP_ZERO_ROWS)
        if ctx.inplace:
            _bwd_(*args)
            return logits, None, None, None, None
        return _bwd(*args), None, None, None, None


_FLOATS = (torch.float32, torch.bfloat16, torch.float16)


def _check_logits(logits):
    """-> (logits the kernels accept, dtype to cast the results to or None)."""
    if not isinstance(logits, torch.Tensor) or logits.dim() < 1:
        raise TypeError("logits must be a tensor of shape (..., vocab_size)")
    if logits.dtype not in _FLOATS and logits.dtype != torch.float64:
        raise TypeError(f"logits dtype {logits.dtype} is not supported (float32, float64, bfloat16, float16)")
    if not logits.is_cuda:
        raise RuntimeError(f"siirl_amd: `logits` is on {logits.device}; these ops run on the GPU only (no CPU fallback)")
    back = None
    if logits.dtype == torch.float64:
        # the reference's fp32 / fp64 branch (torch_functional.py:103-107) serves float64: computed here in fp32
        logits, back = logits.to(torch.float32), torch.float64
    if logits.shape[-1] > 1 and logits.stride(-1) != 1:
        logits = logits.contiguous()
    return logits, back


def logprobs_and_entropy_from_logits(logits: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0,
                                     inplace_backward: bool = False):
    """Both per-token outputs of the actor's post-logits step in one pass: ``(logprob, entropy)`` of
    ``logits / temperature``.  The division is folded into the kernels, ``logits`` is left untouched
    (the reference divides in place first, ``siirl/engine/actor/dp_actor.py:176``)."""
    if torch.compiler.is_compiling():
        return _outside_graph(logprobs_and_entropy_from_logits)(logits, labels, temperature, inplace_backward)
    logits, back = _check_logits(logits)
    lp, ent = _lpe(logits, labels, 1.0 / float(temperature), True, bool(inplace_backward), _SKIP_ZERO_ROWS, None)
    return (lp, ent) if back is None else (lp.to(back), ent.to(back))


def logprob_entropy_traceable(logits: torch.Tensor, labels=None, temperature: float = 1.0, want_entropy: bool = True):
    """``(logprob, entropy)`` as one Python ``autograd.Function`` over the plain ``torch.ops.siirl_hip`` operators
    (opaque to Dynamo, with fake kernels): for a region compiled with ``torch.compile(fullgraph=True)``, where a
    graph break is not allowed.  No pairing state, never in place; an output that was not asked for is empty."""
    if logits.dtype not in _FLOATS:
        raise TypeError(f"logits dtype {logits.dtype} is not supported (float32, bfloat16, float16)")
    return _LogprobEntropy.apply(logits, labels, 1.0 / float(temperature), bool(want_entropy), False)


# Under ``torch.compile`` the reference-named functions below leave the graph for the duration of the call (the
# reference compiles ``entropy_from_logits`` alone, siirl/engine/actor/dp_actor.py:80-84, default ``fullgraph=False``):
# the eager body runs as it would uncompiled, with the pairing and the in-place bookkeeping intact.
_disabled = {}


def _outside_graph(fn):
    wrapped = _disabled.get(fn)
    if wrapped is None:
        wrapped = _disabled[fn] = torch.compiler.disable(fn)
    return wrapped


# ------------------------------------------------------------------------------ pairing
#
# logprobs_from_logits computes the entropy of the same rows in its one pass (the row is in registers anyway) and
# hangs it on the returned log-prob tensor; entropy_from_logits(logits) on the same tensor object, at the same
# version and grad mode, hands it out.  Both then belong to ONE autograd node, which autograd runs once with both
# upstream gradients: one backward pass over the rows, and an in-place backward that cannot overtake a second reader.
# The slot below only holds weak references: the parked entropy lives exactly as long as the log-probs it came with,
# so an unclaimed one pins nothing once the caller drops those.  The slot is per Python thread (the reference's actor
# is one thread per process, a Ray worker per GPU): calls of another thread neither claim nor disturb it.

_PAIRING = True


class _PairingState(threading.local):
    slot = None    # (weakref logits, version, grad mode, weakref entropy or None, defer flag or None, output dtype)
    reader = None  # (weakref to the last separately computed entropy that carries a graph, its logits' storage)


_st = _PairingState()


def set_pairing(flag: bool) -> None:
    global _PAIRING
    _PAIRING, _st.slot, _st.reader = bool(flag), None, None


def _version(t):
    return 0 if t.is_inference() else t._version


def _claim(logits):
    """The parked entropy for exactly this tensor, or None.  A miss on a tensor that shares memory with logits whose
    log-prob node was built for an in-place backward turns that backward out-of-place: the caller is about to give
    those logits a second reader (its own entropy node, or a checkpoint's recomputation), which an in-place backward
    running first would feed with gradients instead of logits."""
    if _st.slot is None:
        return None
    ref, version, grad_mode, ent_ref, defer, back = _st.slot
    parked = ref()
    if parked is None:
        _st.slot = None
        return None
    if ent_ref is not None and parked is logits and _version(logits) == version and \
            torch.is_grad_enabled() == grad_mode:
        ent = ent_ref()
        if ent is not None:
            _st.slot = None
            return ent if back is None else ent.to(back)
    if defer is not None and parked.untyped_storage().data_ptr() == logits.untyped_storage().data_ptr():
        defer[0] = 1
    return None


def _has_reader(logits) -> bool:
    """True while an entropy computed on its own from the same memory is alive with a graph: its node has saved the
    logits, so a log-prob node built now must not overwrite them."""
    if _st.reader is None:
        return False
    ent_ref, storage = _st.reader
    if ent_ref() is None:
        _st.reader = None
        return False
    return storage == logits.untyped_storage().data_ptr()


def _logprobs(logits, labels, inplace_backward, caller_logits, back):
    tracked = logits.requires_grad and torch.is_grad_enabled()
    if inplace_backward and tracked and _has_reader(logits):
        inplace_backward = False
    defer = torch.zeros(1, dtype=torch.int32) if (inplace_backward and tracked) else None
    lp, ent = _lpe(logits, labels, 1.0, _PAIRING, inplace_backward, _SKIP_ZERO_ROWS, defer)
    if _PAIRING:
        lp._siirl_paired_entropy = ent  # keeps the entropy (and through it the node) alive as long as the log-probs
        _st.slot = (weakref.ref(caller_logits), _version(caller_logits), torch.is_grad_enabled(), weakref.ref(ent), defer,
                 back)
    elif defer is not None:
        _st.slot = (weakref.ref(caller_logits), 0, True, None, defer, back)
    return lp


# ------------------------------------------------------------------------------ reference API


def gather_from_labels(data: torch.Tensor, label: torch.Tensor) -> torch.Tensor:
    """reference ``torch_functional.py:41-53`` (plain indexing; not a hot op)."""
    return torch.gather(data, -1, label.unsqueeze(-1)).squeeze(-1)


def logprobs_from_logits(logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = True):
    """Log-probability of ``labels`` under ``softmax(logits)``, shape ``logits.shape[:-1]``
    (reference ``torch_functional.py:56-82``).  With ``inplace_backward=True`` the backward pass
    overwrites ``logits`` with its gradient, as the reference's flash-attn path does (``:85-90``)."""
    if torch.compiler.is_compiling():
        return _outside_graph(logprobs_from_logits)(logits, labels, inplace_backward)
    x, back = _check_logits(logits)
    # a converted copy (fp64, non-unit vocab stride) is private to this call: nothing to overwrite in place
    lp = _logprobs(x, labels, bool(inplace_backward) and x is logits, logits, back)
    return lp if back is None else lp.to(back)


def logprobs_from_logits_v2(logits: torch.Tensor, labels: torch.Tensor):
    """reference ``torch_functional.py:99-116``; same kernel, never in place, nothing parked."""
    if torch.compiler.is_compiling():
        return _outside_graph(logprobs_from_logits_v2)(logits, labels)
    x, back = _check_logits(logits)
    lp, _ = _lpe(x, labels, 1.0, False, False, _SKIP_ZERO_ROWS, None)
    return lp if back is None else lp.to(back)


logprobs_from_logits_naive = logprobs_from_logits_v2  # reference :93-96


def logprobs_from_logits_flash_attn(logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = True):
    """reference ``torch_functional.py:85-90`` (the negated flash-attn cross-entropy): fp32 log-probs of 2-D
    ``logits`` whatever their dtype, 0 for a label of -100, backward in place when ``inplace_backward``."""
    if logits.dim() != 2 or labels.dim() != 1:
        raise ValueError("siirl_amd: logprobs_from_logits_flash_attn takes [tokens, vocab] logits and [tokens] labels")
    return logprobs_from_logits(logits, labels, inplace_backward=inplace_backward)


def entropy_from_logits(logits: torch.Tensor):
    """Entropy of ``softmax(logits)`` per row (reference ``torch_functional.py:128-132``)."""
    if torch.compiler.is_compiling():
        return _outside_graph(entropy_from_logits)(logits)
    x, back = _check_logits(logits)
    parked = _claim(logits)
    if parked is not None:
        return parked
    _, ent = _lpe(x, None, 1.0, True, False, _SKIP_ZERO_ROWS, None)
    if ent.requires_grad:
        _st.reader = (weakref.ref(ent), x.untyped_storage().data_ptr())
    return ent if back is None else ent.to(back)


def entropy_from_logits_with_chunking(logits: torch.Tensor, chunk_size: int = 2048):
    """reference ``torch_functional.py:135-143``.  The chunking there bounds the fp32 temporaries; the
    kernel has none, so the whole tensor goes in one launch.  2-D input, fp32 output, as there."""
    if logits.dim() != 2:
        raise ValueError("entropy_from_logits_with_chunking expects a 2-D tensor")
    ent = entropy_from_logits(logits)
    return ent if ent.dtype == torch.float32 else ent.to(torch.float32)


# ------------------------------------------------------------------------------ masked reductions


def _masked_reduce(values: torch.Tensor, mask: torch.Tensor, axis, want_mean: bool):
    if not values.is_cuda:
        raise RuntimeError("siirl_amd: masked reductions run on the GPU only (no CPU fallback)")
    if axis is None:
        axes = []
    elif isinstance(axis, (tuple, list)):
        axes = [int(a) for a in axis]
        if not axes:  # torch's sum over an empty tuple of axes reduces everything
            axes = list(range(values.dim()))
    else:
        axes = [int(axis)]
    if axis is not None and values.dim() and len(set(a % values.dim() for a in axes)) == values.dim():
        axes = []
    return _OPS.masked_reduce(values, mask, axes, want_mean)


def masked_sum(values: torch.Tensor, mask: torch.Tensor, axis=None):
    """``sum(where(mask, values, 0) * mask)`` over everything or over ``axis`` (an int or a tuple of ints;
    reference ``torch_functional.py:146-151``); fp32 result, differentiable in ``values``."""
    return _masked_reduce(values, mask, axis, want_mean=False)


def masked_mean(values: torch.Tensor, mask: torch.Tensor, axis=None):
    """``masked_sum / (mask.sum(axis) + 1e-8)`` (reference ``torch_functional.py:154-168``); differentiable in
    ``values``."""
    return _masked_reduce(values, mask, axis, want_mean=True)


def clip_by_value(x: torch.Tensor, tensor_min: torch.Tensor, tensor_max: torch.Tensor):
    """``max(min(x, tensor_max), tensor_min)`` with tensor bounds (reference ``torch_functional.py:119-125``);
    plain torch, it is not on the hot path by itself (the value loss fuses it)."""
    return torch.max(torch.min(x, tensor_max), tensor_min)


def _check_whiten_count(n: float):
    """The two ``ValueError``s of the reference's ``masked_var`` (``torch_functional.py:178-184``)."""
    if n == 0:
        raise ValueError("At least one element in the mask has to be 1.")
    if n == 1:
        raise ValueError("The sum of the mask is one, which can cause a division by zero.")


def _whiten(values: torch.Tensor, mask: torch.Tensor, shift_mean: bool):
    from . import _lib
    from . import core_algos as CA

    if not values.is_cuda:
        raise RuntimeError("siirl_amd: masked_var / masked_whiten run on the GPU only (no CPU fallback)")
    dev = values.device
    v = CA._f32(values, dev)
    m, mcode = CA._mask_arg(mask.expand_as(values), dev)
    out = torch.empty_like(v)
    stats = torch.empty(3, dtype=torch.float32, device=dev)
    nws = _lib.lib().siirl_whiten_workspace_bytes()
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_masked_whiten(_lib.ptr(v), _lib.ptr(m), mcode, v.numel(), int(bool(shift_mean)),
                                            _lib.ptr(out), _lib.ptr(stats), _lib.ptr(ws), nws,
                                            _lib.current_stream(dev))
    _lib.check(rc, "siirl_masked_whiten")
    return out, stats


def masked_var(values: torch.Tensor, mask: torch.Tensor, unbiased: bool = True):
    """Variance over the masked elements (reference ``torch_functional.py:171-187``), 0-d fp32.  The biased form of
    a mask that selects one element, or none, is 0 as there (``masked_mean`` of zeros, or ``0 / 1e-8``)."""
    _, stats = _whiten(values, mask, True)
    n = float(stats[2])
    if unbiased:
        _check_whiten_count(n)
        return stats[1]
    return stats[1] * ((n - 1.0) / n) if n > 1 else torch.zeros_like(stats[1])


def masked_whiten(values: torch.Tensor, mask: torch.Tensor, shift_mean: bool = True):
    """``(values - mean) * rsqrt(var + 1e-8)`` with masked mean and unbiased masked variance, applied to every
    element (reference ``torch_functional.py:190-206``); no gradient (the reference uses it under ``no_grad``)."""
    out, stats = _whiten(values, mask, shift_mean)
    _check_whiten_count(float(stats[2]))
    return out.reshape(values.shape)


# ------------------------------------------------------------------------------ response masks and rmpad glue


def get_response_mask(response_id: torch.Tensor, eos_token=2, dtype=torch.int64):
    """1 up to and including the first end-of-sequence token of each row, 0 after it; ``eos_token`` is an int or a
    list of ints (reference ``torch_functional.py:209-229``: ``(cumsum(isin) - isin) == 0``)."""
    if not response_id.is_cuda:
        raise RuntimeError(f"siirl_amd: `response_id` is on {response_id.device}; these ops run on the GPU only")
    if response_id.dim() != 2:
        raise ValueError(f"response_id must be [batch, response_length], got {tuple(response_id.shape)}")
    if response_id.dtype not in (torch.int64, torch.int32):
        raise TypeError(f"response_id dtype {response_id.dtype} is not supported (int64, int32)")
    import ctypes

    from . import _lib

    toks = [int(t) for t in (eos_token if isinstance(eos_token, (list, tuple)) else [eos_token])]
    if len(toks) > _lib.MAX_EOS_TOKENS:
        raise ValueError(f"at most {_lib.MAX_EOS_TOKENS} end-of-sequence tokens are supported, got {len(toks)}")
    ids = response_id.contiguous()
    B, L = ids.shape
    out_dtype = torch.uint8 if dtype == torch.bool else dtype
    out = torch.empty(B, L, dtype=out_dtype, device=ids.device)
    arr = (ctypes.c_int64 * max(len(toks), 1))(*toks)
    with torch.cuda.device(ids.device):
        rc = _lib.lib().siirl_eos_response_mask(_lib.ptr(ids), _lib.dtype_code(ids.dtype), B, L, arr, len(toks),
                                                _lib.ptr(out), _lib.dtype_code(out_dtype),
                                                _lib.current_stream(ids.device))
    _lib.check(rc, "siirl_eos_response_mask")
    return out.view(torch.bool) if dtype == torch.bool else out


def get_eos_mask(response_id: torch.Tensor, eos_token: int = 2, dtype=torch.int64):
    """The single-token form (reference ``torch_functional.py:232-254``); same mask."""
    return get_response_mask(response_id, int(eos_token), dtype)


def get_unpad_data(attention_mask: torch.Tensor):
    """``(indices, cu_seqlens, max_seqlen_in_batch)`` of the attended positions (reference
    ``torch_functional.py:638-647``)."""
    from . import padding

    indices, cu, max_seqlen, _ = padding._unpad_indices(attention_mask)
    return indices, cu, max_seqlen


def log_probs_from_logits_response(input_ids, logits, response_length):
    """Log-probs of the response tokens from padded logits ``[batch, seqlen, vocab]`` (reference
    ``torch_functional.py:431-444``).  The ``[:, -response_length - 1 : -1]`` window is read in place through its
    row stride; no copy of the logits is made."""
    response_logits = logits[:, -response_length - 1:-1]
    response = input_ids[:, -response_length:]
    return logprobs_from_logits(logits=response_logits, labels=response)


def log_probs_from_logits_all_rmpad(input_ids_rmpad, logits_rmpad, indices, batch_size, seqlen, response_length):
    """Response log-probs ``[batch, response_length]`` from packed ids ``[1, nnz]`` and packed logits
    ``[nnz, vocab]`` (reference ``torch_functional.py:474-500``): labels are the ids rolled by one, the packed
    log-probs are scattered straight into the response window."""
    from . import padding

    ids = input_ids_rmpad.reshape(-1)
    rolled = torch.roll(ids, shifts=-1, dims=0)
    full_log_probs_rmpad = logprobs_from_logits(logits=logits_rmpad, labels=rolled)
    return padding.pad_and_slice_response(full_log_probs_rmpad, indices, batch_size, seqlen, response_length)


def log_probs_from_logits_response_rmpad(input_ids, attention_mask, logits_rmpad, response_length):
    """Same result from padded ids ``[batch, seqlen]`` + attention mask and packed logits (reference
    ``torch_functional.py:447-471``)."""
    from . import padding

    batch_size, seqlen = input_ids.shape
    _, rolled, indices, _, _ = padding.unpad_ids_and_labels(input_ids, attention_mask)
    full_log_probs_rmpad = logprobs_from_logits(logits=logits_rmpad, labels=rolled)
    return padding.pad_and_slice_response(full_log_probs_rmpad, indices, batch_size, seqlen, response_length)


def remove_pad_token(input_ids: torch.Tensor, attention_mask: torch.Tensor):
    """Per-row python lists of the last ``mask.sum()`` ids (reference ``torch_functional.py:416-428``); host-side
    list building, one device-to-host copy for the whole batch."""
    ids = input_ids.cpu()
    counts = attention_mask.sum(dim=-1).cpu().tolist()
    return [row[len(row) - int(n):].numpy().tolist() for row, n in zip(ids, counts)]
