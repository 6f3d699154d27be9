"""Oracle (test infrastructure): remove-padding bookkeeping around the log-prob computation.

The reference calls flash-attn's ``bert_padding`` helpers (``unpad_input``, ``index_first_axis``, ``pad_input``;
flash-attn 2.7.3 / 2.8.2, a third-party dependency that is not in the reference tree) at
``siirl/engine/actor/dp_actor.py:112-127,214-231``.  Their published algorithm is restated here in numpy:
``indices = nonzero(mask.flatten())``, ``cu_seqlens = [0, cumsum(mask.sum(-1))]``, gather / zero-filled scatter
along the first axis; plus the reference's own ``torch.roll(input_ids_rmpad, -1)`` labels and the
``[:, -response_length - 1 : -1]`` response window.  Integer work: parity is exact."""

from __future__ import annotations

import numpy as np


def unpad_input(hidden_states: np.ndarray, attention_mask: np.ndarray):
    """``hidden_states [B, S, ...]``, 0/1 ``attention_mask [B, S]`` -> ``(hidden_rmpad [nnz, ...], indices [nnz],
    cu_seqlens [B + 1] int32, max_seqlen, seqlens [B] int32)`` (the 5-tuple of flash-attn >= 2.7)."""
    B, S = attention_mask.shape
    seqlens = (attention_mask != 0).sum(axis=-1).astype(np.int32)
    indices = np.flatnonzero(attention_mask.reshape(-1)).astype(np.int64)
    cu = np.concatenate([[0], np.cumsum(seqlens)]).astype(np.int32)
    flat = hidden_states.reshape((B * S,) + hidden_states.shape[2:])
    return flat[indices], indices, cu, int(seqlens.max()), seqlens


def index_first_axis(x: np.ndarray, indices: np.ndarray):
    return x[indices]


def pad_input(hidden_states: np.ndarray, indices: np.ndarray, batch: int, seqlen: int):
    """Zero-filled ``[batch, seqlen, ...]`` with ``hidden_states[j]`` at flat position ``indices[j]``."""
    out = np.zeros((batch * seqlen,) + hidden_states.shape[1:], dtype=hidden_states.dtype)
    out[indices] = hidden_states
    return out.reshape((batch, seqlen) + hidden_states.shape[1:])


def rolled_labels(input_ids_rmpad: np.ndarray):
    """``torch.roll(input_ids_rmpad, shifts=-1)`` (reference ``dp_actor.py:127``): token j is scored against
    token j + 1; the last wraps to the first."""
    return np.roll(input_ids_rmpad, -1)


def pad_and_slice_response(values_rmpad: np.ndarray, indices: np.ndarray, batch: int, seqlen: int,
                           response_length: int):
    """``pad_input(values.unsqueeze(-1), ...).squeeze(-1)[:, -response_length - 1 : -1]`` (reference
    ``dp_actor.py:214-231``)."""
    full = pad_input(values_rmpad[:, None], indices, batch, seqlen)[..., 0]
    return full[:, -response_length - 1:-1]
