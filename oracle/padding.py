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


def get_response_mask(response_id: np.ndarray, eos_token=2, dtype=np.int64):
    """1 up to and including the first end-of-sequence token of each row, 0 after (reference
    ``siirl/utils/model_utils/torch_functional.py:209-229``, which writes it as ``(cumsum(isin) - isin) == 0``;
    ``get_eos_mask`` at ``:232-254`` is the single-token case).  Pinned by the two worked examples of the
    reference's docstring (``tests/test_oracle_padding.py``)."""
    eos = set(np.atleast_1d(np.asarray(eos_token)).tolist())
    out = np.zeros(response_id.shape, dtype=dtype)
    for b, row in enumerate(response_id.tolist()):
        for t, tok in enumerate(row):
            out[b, t] = 1
            if tok in eos:
                break
    return out


def get_unpad_data(attention_mask: np.ndarray):
    """``(indices, cu_seqlens, max_seqlen_in_batch)`` (reference ``torch_functional.py:638-647``)."""
    _, indices, cu, max_seqlen, _ = unpad_input(attention_mask[..., None], attention_mask)
    return indices, cu, max_seqlen


def remove_pad_token(input_ids: np.ndarray, attention_mask: np.ndarray):
    """Per-row lists of the last ``mask.sum()`` ids (reference ``torch_functional.py:416-428``)."""
    return [row[len(row) - int(m.sum()):].tolist() for row, m in zip(input_ids, attention_mask)]
