"""Remove-padding helpers with the names and return values the reference's actor uses.

Mirror of what ``siirl/engine/actor/dp_actor.py:112-127,214-231`` imports from flash-attn's ``bert_padding``
(``unpad_input``, ``index_first_axis``, ``pad_input``) plus two fusions of the surrounding lines:
``unpad_ids_and_labels`` (packed ids and the rolled next-token labels in one pass) and
``pad_and_slice_response`` (``pad_input`` + the ``[:, -response_length - 1 : -1]`` window without the padded
``[B, S]`` intermediate).  The index arithmetic runs in ``libsiirl_hip.so``; tensors must be on the GPU."""

from __future__ import annotations

import torch

from . import _lib

__all__ = ["unpad_input", "index_first_axis", "pad_input", "unpad_ids_and_labels", "pad_and_slice_response"]


LABEL_SKIP_ROW = _lib.LABEL_SKIP_ROW  # label of a packed row that the log-prob kernels skip


def _need_gpu(t: torch.Tensor, name: str):
    if not t.is_cuda:
        raise RuntimeError(f"siirl_amd: `{name}` is on {t.device}; these ops run on the GPU only (no CPU fallback)")


def _mask_arg(mask: torch.Tensor):
    m = mask.detach()
    if m.dtype not in (torch.bool, torch.uint8, torch.int32, torch.int64, torch.float32, torch.bfloat16, torch.float16):
        m = m.to(torch.int32)
    m = m.contiguous()
    return m, _lib.dtype_code(m.dtype)


def _unpad_indices(attention_mask: torch.Tensor):
    _need_gpu(attention_mask, "attention_mask")
    if attention_mask.dim() != 2:
        raise ValueError(f"attention_mask must be [batch, seqlen], got {tuple(attention_mask.shape)}")
    B, S = attention_mask.shape
    dev = attention_mask.device
    m, mcode = _mask_arg(attention_mask)
    seqlens = torch.empty(B, dtype=torch.int32, device=dev)
    cu = torch.empty(B + 1, dtype=torch.int32, device=dev)
    indices = torch.empty(B * S, dtype=torch.int64, device=dev)
    info = torch.empty(2, dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().siirl_unpad_indices(_lib.ptr(m), mcode, B, S, _lib.ptr(seqlens), _lib.ptr(cu),
                                            _lib.ptr(indices), _lib.ptr(info), _lib.current_stream(dev))
    _lib.check(rc, "siirl_unpad_indices")
    nnz, max_seqlen = info.tolist()  # the one host sync; the reference's .item() for max_seqlen is the same
    return indices[:nnz], cu, int(max_seqlen), seqlens


def _rows(x: torch.Tensor):
    row_bytes = x[0].numel() * x.element_size() if x.shape[0] else 0
    if x.shape[0] and (row_bytes < 4 or row_bytes % 4):
        raise ValueError(f"rows of {row_bytes} bytes: index_first_axis / pad_input move whole 4-byte words")
    return row_bytes


class _IndexFirstAxis(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, indices):
        _need_gpu(x, "input")
        x = x.contiguous()
        n = indices.numel()
        out = torch.empty((n,) + x.shape[1:], dtype=x.dtype, device=x.device)
        ctx.save_for_backward(indices)
        ctx.total = x.shape[0]
        if n:
            with torch.cuda.device(x.device):
                rc = _lib.lib().siirl_gather_rows(_lib.ptr(x), _lib.ptr(indices), n, _rows(x), x.shape[0],
                                                  _lib.ptr(out), _lib.current_stream(x.device))
            _lib.check(rc, "siirl_gather_rows")
        return out

    @staticmethod
    def backward(ctx, g):
        (indices,) = ctx.saved_tensors
        return _PadRows.apply(g, indices, ctx.total), None


class _PadRows(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, indices, total):
        _need_gpu(x, "hidden_states")
        x = x.contiguous()
        n = indices.numel()
        out = torch.empty((total,) + x.shape[1:], dtype=x.dtype, device=x.device)
        ctx.save_for_backward(indices)
        row_bytes = _rows(x) if n else out[0].numel() * out.element_size()
        with torch.cuda.device(x.device):
            rc = _lib.lib().siirl_scatter_rows(_lib.ptr(x), _lib.ptr(indices), n, row_bytes, total, _lib.ptr(out),
                                               _lib.current_stream(x.device))
        _lib.check(rc, "siirl_scatter_rows")
        return out

    @staticmethod
    def backward(ctx, g):
        (indices,) = ctx.saved_tensors
        return _IndexFirstAxis.apply(g, indices), None, None


def index_first_axis(x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """``x[indices]`` along the first axis, differentiable (flash-attn ``bert_padding.index_first_axis``)."""
    return _IndexFirstAxis.apply(x, indices.to(torch.int64).contiguous())


def unpad_input(hidden_states: torch.Tensor, attention_mask: torch.Tensor, unused_mask=None):
    """``(hidden_states_rmpad [nnz, ...], indices [nnz], cu_seqlens [B + 1] int32, max_seqlen_in_batch, seqlens
    [B] int32)`` for a 0/1 ``attention_mask [B, S]`` -- the 5-tuple of flash-attn >= 2.7 ``bert_padding.unpad_input``
    (the reference unpacks ``x, indices, cu_seqlens, *_``, ``dp_actor.py:112``)."""
    if unused_mask is not None:
        raise NotImplementedError("unused_mask is outside this build")
    indices, cu, max_seqlen, seqlens = _unpad_indices(attention_mask)
    B, S = attention_mask.shape
    flat = hidden_states.reshape((B * S,) + tuple(hidden_states.shape[2:]))
    return index_first_axis(flat, indices), indices, cu, max_seqlen, seqlens


def pad_input(hidden_states: torch.Tensor, indices: torch.Tensor, batch: int, seqlen: int) -> torch.Tensor:
    """Zero-filled ``[batch, seqlen, ...]`` holding ``hidden_states[j]`` at flat position ``indices[j]``
    (flash-attn ``bert_padding.pad_input``), differentiable."""
    out = _PadRows.apply(hidden_states, indices.to(torch.int64).contiguous(), batch * seqlen)
    return out.reshape((batch, seqlen) + tuple(hidden_states.shape[1:]))


def unpad_ids_and_labels(input_ids: torch.Tensor, attention_mask: torch.Tensor, response_length: int = None):
    """``(input_ids_rmpad [1, nnz], input_ids_rmpad_rolled [nnz], indices, cu_seqlens, max_seqlen)``: the packed ids
    and ``torch.roll(input_ids_rmpad, -1)`` of reference ``dp_actor.py:112-127`` from one kernel.

    With ``response_length`` the rolled labels of the packed tokens outside each sequence's response window (the
    positions the slice ``[:, -response_length - 1 : -1]`` of ``dp_actor.py:228-231`` drops) are set to
    ``LABEL_SKIP_ROW``: ``logprobs_from_logits`` / ``entropy_from_logits`` then neither read those rows of the
    packed logits nor send a gradient into them, and return 0 there; what the window keeps is unchanged."""
    _need_gpu(input_ids, "input_ids")
    indices, cu, max_seqlen, _ = _unpad_indices(attention_mask)
    ids = input_ids.to(torch.int64).contiguous()
    nnz = indices.numel()
    rm = torch.empty(nnz, dtype=torch.int64, device=ids.device)
    rolled = torch.empty(nnz, dtype=torch.int64, device=ids.device)
    with torch.cuda.device(ids.device):
        rc = _lib.lib().siirl_unpad_ids_labels(_lib.ptr(ids), ids.numel(), _lib.ptr(indices), nnz, _lib.ptr(rm),
                                               _lib.ptr(rolled), _lib.current_stream(ids.device))
    _lib.check(rc, "siirl_unpad_ids_labels")
    if response_length is not None:
        S = attention_mask.shape[1]
        with torch.cuda.device(ids.device):
            rc = _lib.lib().siirl_mark_rows_outside_response(_lib.ptr(indices), nnz, S, int(response_length),
                                                             _lib.ptr(rolled), _lib.current_stream(ids.device))
        _lib.check(rc, "siirl_mark_rows_outside_response")
    return rm.unsqueeze(0), rolled, indices, cu, max_seqlen


class _ResponseWindow(torch.autograd.Function):
    @staticmethod
    def forward(ctx, values, indices, B, S, L):
        _need_gpu(values, "values")
        v = values.detach().to(torch.float32).contiguous()
        out = torch.empty(B, L, dtype=torch.float32, device=v.device)
        with torch.cuda.device(v.device):
            rc = _lib.lib().siirl_response_scatter(_lib.ptr(v), _lib.ptr(indices), v.numel(), B, S, L, _lib.ptr(out),
                                                   _lib.current_stream(v.device))
        _lib.check(rc, "siirl_response_scatter")
        ctx.save_for_backward(indices)
        ctx.meta = (S, L, values.dtype)
        return out.to(values.dtype)

    @staticmethod
    def backward(ctx, g):
        (indices,) = ctx.saved_tensors
        S, L, dtype = ctx.meta
        g = g.detach().to(torch.float32).contiguous()
        d = torch.empty(indices.numel(), dtype=torch.float32, device=g.device)
        with torch.cuda.device(g.device):
            rc = _lib.lib().siirl_response_gather(_lib.ptr(g), _lib.ptr(indices), indices.numel(), g.shape[0], S, L,
                                                  _lib.ptr(d), _lib.current_stream(g.device))
        _lib.check(rc, "siirl_response_gather")
        return d.to(dtype), None, None, None, None


def pad_and_slice_response(values_rmpad: torch.Tensor, indices: torch.Tensor, batch: int, seqlen: int,
                           response_length: int) -> torch.Tensor:
    """``pad_input(values_rmpad.unsqueeze(-1), indices, batch, seqlen).squeeze(-1)[:, -response_length - 1 : -1]``
    (reference ``dp_actor.py:214-231``) as one scatter into the ``[batch, response_length]`` result; differentiable."""
    if values_rmpad.dim() != 1 or values_rmpad.numel() != indices.numel():
        raise ValueError(f"values {tuple(values_rmpad.shape)} must be [nnz] with nnz = {indices.numel()}")
    if not 1 <= response_length <= seqlen - 1:
        raise ValueError(f"response_length {response_length} must be in [1, seqlen - 1 = {seqlen - 1}]")
    return _ResponseWindow.apply(values_rmpad, indices.to(torch.int64).contiguous(), batch, seqlen, response_length)
