"""Pins the oracle's remove-padding restatement (CPU only) against the pure-torch statement of flash-attn's
bert_padding that ships in transformers, a round trip, and a hand-written case."""
import numpy as np
import pytest
import torch

from oracle import padding as OP


def _case(B, S, seed):
    rng = np.random.default_rng(seed)
    left = rng.integers(0, S // 2, B)
    right = rng.integers(0, S // 2, B)
    mask = np.zeros((B, S), dtype=np.int64)
    for b in range(B):
        mask[b, left[b]:S - right[b]] = 1
    mask[0, :] = 1
    ids = rng.integers(0, 50000, (B, S)).astype(np.int64)
    return ids, mask


def test_hand_written_case():
    mask = np.array([[0, 1, 1, 0], [1, 1, 1, 1], [0, 0, 0, 1]])
    x = np.arange(12).reshape(3, 4, 1)
    rm, idx, cu, mx, sl = OP.unpad_input(x, mask)
    assert idx.tolist() == [1, 2, 4, 5, 6, 7, 11] and cu.tolist() == [0, 2, 6, 7] and mx == 4 and sl.tolist() == [2, 4, 1]
    assert rm[:, 0].tolist() == [1, 2, 4, 5, 6, 7, 11]
    assert OP.rolled_labels(rm[:, 0]).tolist() == [2, 4, 5, 6, 7, 11, 1]
    full = OP.pad_input(rm, idx, 3, 4)[..., 0]
    assert full.tolist() == [[0, 1, 2, 0], [4, 5, 6, 7], [0, 0, 0, 11]]
    # response_length 2 of seqlen 4: columns 1 and 2
    assert OP.pad_and_slice_response(rm[:, 0].astype(np.float32), idx, 3, 4, 2).tolist() == [[1, 2], [5, 6], [0, 0]]


@pytest.mark.parametrize("B,S", [(1, 2), (4, 37), (16, 512)])
def test_against_transformers_restatement(B, S):
    mfu = pytest.importorskip("transformers.modeling_flash_attention_utils")
    ids, mask = _case(B, S, B * S)
    h = np.random.default_rng(1).standard_normal((B, S, 3)).astype(np.float32)
    rm, idx, cu, mx, sl = OP.unpad_input(h, mask)
    t_rm, t_idx, t_cu, t_mx, t_sl = mfu._unpad_input(torch.from_numpy(h), torch.from_numpy(mask))
    assert np.array_equal(rm, t_rm.numpy()) and np.array_equal(idx, t_idx.numpy())
    assert np.array_equal(cu, t_cu.numpy()) and mx == t_mx and np.array_equal(sl, t_sl.numpy())
    assert np.array_equal(OP.pad_input(rm, idx, B, S), mfu._pad_input(t_rm, t_idx, B, S).numpy())
    assert np.array_equal(OP.index_first_axis(h.reshape(B * S, 3), idx), rm)


@pytest.mark.parametrize("B,S,L", [(3, 9, 4), (8, 300, 128), (2, 5, 4)])
def test_round_trip_and_window(B, S, L):
    ids, mask = _case(B, S, S)
    v = np.random.default_rng(2).standard_normal((B, S)).astype(np.float32)
    rm, idx, *_ = OP.unpad_input(v[..., None], mask)
    assert np.array_equal(OP.pad_input(rm, idx, B, S)[..., 0], v * mask)
    assert np.array_equal(OP.pad_and_slice_response(rm[:, 0], idx, B, S, L), (v * mask)[:, S - L - 1:S - 1])


def test_response_mask_docstring_examples_of_the_reference():
    """The two worked examples in the docstring of get_response_mask and the one of get_eos_mask
    (reference siirl/utils/model_utils/torch_functional.py:212-226, 236-238)."""
    ids = np.array([[20, 10, 34, 1, 0, 0, 0], [78, 0, 76, 2, 1, 0, 0], [23, 98, 1, 0, 0, 0, 0], [33, 3, 98, 45, 1, 0, 0]])
    assert OP.get_response_mask(ids, 1).tolist() == [[1, 1, 1, 1, 0, 0, 0], [1, 1, 1, 1, 1, 0, 0], [1, 1, 1, 0, 0, 0, 0],
                                                     [1, 1, 1, 1, 1, 0, 0]]
    assert OP.get_response_mask(ids, [1, 2]).tolist() == [[1, 1, 1, 1, 0, 0, 0], [1, 1, 1, 1, 0, 0, 0],
                                                          [1, 1, 1, 0, 0, 0, 0], [1, 1, 1, 1, 1, 0, 0]]
    assert OP.get_response_mask(np.array([[0, 0, 2, 42, 3, 5, 1, 0, 0]]), 1).tolist() == [[1, 1, 1, 1, 1, 1, 1, 0, 0]]
    # the closed form the reference uses, on random rows
    rng = np.random.default_rng(0)
    ids = rng.integers(0, 6, (50, 33))
    isin = np.isin(ids, [2, 5]).astype(np.int64)
    assert np.array_equal(OP.get_response_mask(ids, [2, 5]), ((np.cumsum(isin, axis=1) - isin) == 0).astype(np.int64))
    assert OP.get_response_mask(ids, 77).all()


def test_unpad_data_and_remove_pad_token():
    mask = np.array([[0, 1, 1, 1], [0, 0, 0, 1], [1, 1, 1, 1]])
    idx, cu, mx = OP.get_unpad_data(mask)
    assert idx.tolist() == [1, 2, 3, 7, 8, 9, 10, 11] and cu.tolist() == [0, 3, 4, 8] and mx == 4
    ids = np.arange(12).reshape(3, 4)
    assert OP.remove_pad_token(ids, mask) == [[1, 2, 3], [7], [8, 9, 10, 11]]


def test_rmpad_response_logprobs_equal_the_padded_form():
    """Where the response window and the position before it are attended, the packed route gives the padded
    route's numbers: row j of the packed logits is position indices[j] of the padded ones."""
    from oracle import torch_functional as OT

    B, S, L, V = 3, 12, 4, 29
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(B, S, V, generator=g)
    ids = torch.randint(0, V, (B, S), generator=g)
    mask = torch.ones(B, S, dtype=torch.int64)
    mask[0, :5] = 0
    mask[2, :2] = 0
    want = OT.log_probs_from_logits_response(ids, logits, L)
    idx = torch.nonzero(mask.flatten()).flatten()
    packed = logits.reshape(B * S, V)[idx]
    got = OT.log_probs_from_logits_response_rmpad(ids, mask, packed, L)
    assert got.shape == (B, L) and torch.allclose(got, want, atol=1e-6)
    got2 = OT.log_probs_from_logits_all_rmpad(ids.flatten()[idx][None], packed, idx, B, S, L)
    assert torch.equal(got, got2)
    # and the padded form is the textbook log-softmax pick
    ref = torch.log_softmax(logits[:, S - L - 1:S - 1], -1).gather(-1, ids[:, S - L:, None])[..., 0]
    assert torch.allclose(want, ref, atol=1e-6)
