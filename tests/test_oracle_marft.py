"""Pins of the oracle's multi-agent GAE (``oracle.core_algos.marft_gae_unwhitened`` /
``compute_marft_gae_advantage_return``, restating ``siirl/dag_worker/core_algos.py:351-458``) on the CPU:
a two-agent, two-step request worked by hand; the single-agent case against the (separately pinned) GAE scan;
the closed form at gamma = lam = 1; the reference's bookkeeping (id list, keys written, dtypes, errors)."""

from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import core_algos as OC


def _hand_case(mask_dtype=torch.int64):
    # one request of two rows (its last step first); agent 0 answers with up to 2 tokens, the last agent with up to 3
    v0 = torch.tensor([[2.0, 99.0], [4.0, 12.0]])
    r0 = torch.tensor([[32.0, 77.0], [5.0, 8.0]])  # r0[1, 0] = 5 is not at an agent's last token: never read
    m0 = torch.tensor([[1, 0], [1, 1]], dtype=mask_dtype)
    v1 = torch.tensor([[8.0, 4.0, 99.0], [16.0, 8.0, 4.0]])
    r1 = torch.tensor([[3.0, 16.0, 77.0], [0.0, 0.0, 64.0]])  # r1[0, 0] = 3: never read
    m1 = torch.tensor([[1, 1, 0], [1, 1, 1]], dtype=mask_dtype)
    return [r0, r1], [v0, v1], [m0, m1]


# gamma = lam = 0.5 (every product exact in binary), walked by hand:
#   row 0, last agent:  t=1: delta = 16 + .5*0 - 4 = 12,            gae = 12
#                       t=0: delta = .5*4 - 8 = -6,                 gae = -6 + .25*12 = -3
#   row 0, agent 0:     t=0: delta = 32 + .5*8 - 2 = 34,            gae = 34 + .25*(-3) = 33.25
#   row 1, last agent:  t=2: delta = 64 + .5*2 - 4 = 61,            gae = 61 + .25*33.25 = 69.3125
#                       t=1: delta = .5*4 - 8 = -6,                 gae = -6 + .25*69.3125 = 11.328125
#                       t=0: delta = .5*8 - 16 = -12,               gae = -12 + .25*11.328125 = -9.16796875
#   row 1, agent 0:     t=1: delta = 8 + .5*16 - 12 = 4,            gae = 4 + .25*(-9.16796875) = 1.7080078125
#                       t=0: delta = .5*12 - 4 = 2,                 gae = 2 + .25*1.7080078125 = 2.427001953125
HAND_ADV0 = [[33.25, 0.0], [2.427001953125, 1.7080078125]]
HAND_ADV1 = [[-3.0, 12.0, 0.0], [-9.16796875, 11.328125, 69.3125]]
HAND_RET0 = [[35.25, 0.0], [6.427001953125, 13.7080078125]]
HAND_RET1 = [[5.0, 16.0, 0.0], [6.83203125, 19.328125, 73.3125]]


def test_hand_worked_request_in_float_and_truncated():
    r, v, m = _hand_case()
    adv, ret = OC.marft_gae_unwhitened(r, v, m, [(0, 2)], 0.5, 0.5, out_dtype=torch.float32)
    assert adv[0].tolist() == HAND_ADV0 and adv[1].tolist() == HAND_ADV1
    assert ret[0].tolist() == HAND_RET0 and ret[1].tolist() == HAND_RET1
    # the reference's outputs take the (integer) mask's dtype: integer parts, towards zero
    adv, ret = OC.marft_gae_unwhitened(r, v, m, [(0, 2)], 0.5, 0.5)
    assert adv[0].dtype == torch.int64 and ret[1].dtype == torch.int64
    assert adv[0].tolist() == [[33, 0], [2, 1]] and adv[1].tolist() == [[-3, 12, 0], [-9, 11, 69]]
    assert ret[0].tolist() == [[35, 0], [6, 13]] and ret[1].tolist() == [[5, 16, 0], [6, 19, 73]]
    # two requests of one row each: the accumulator restarts and no row looks at the row before
    adv2, _ = OC.marft_gae_unwhitened(r, v, m, [(0, 1), (1, 1)], 0.5, 0.5, out_dtype=torch.float32)
    assert adv2[0][0].tolist() == HAND_ADV0[0] and adv2[1][0].tolist() == HAND_ADV1[0]
    # row 1 alone: last agent t=2: 64 - 4 = 60; t=1: -6 + 15 = 9; t=0: -12 + 2.25 = -9.75; agent 0: 4 - 2.4375, ...
    assert adv2[1][1].tolist() == [-9.75, 9.0, 60.0]
    assert adv2[0][1].tolist() == [2.0 + 0.25 * 1.5625, 1.5625]


def test_single_agent_rows_are_the_gae_scan():
    """With the other agent silent (empty mask), one row per request, full rows and a reward at the last token only,
    the walk is the ordinary GAE recurrence."""
    g = torch.Generator().manual_seed(3)
    B, L = 5, 9
    v = torch.randn(B, L, generator=g)
    r = torch.zeros(B, L)
    r[:, -1] = torch.randn(B, generator=g)
    m = torch.ones(B, L, dtype=torch.int64)
    silent = torch.zeros(B, 2, dtype=torch.int64)
    junk = torch.randn(B, 2, generator=g)
    adv, ret = OC.marft_gae_unwhitened([junk, r], [junk, v], [silent, m], [(b, 1) for b in range(B)], 0.9, 0.95,
                                       out_dtype=torch.float32)
    want_a, want_r = OC.gae_unwhitened(r, v, m.float(), 0.9, 0.95)
    assert torch.equal(adv[1], want_a) and torch.equal(ret[1], want_r)
    assert not adv[0].any() and not ret[0].any()


def test_closed_form_at_gamma_lam_one():
    """gamma = lam = 1: the deltas telescope, so a token's advantage is the sum of the rewards met so far on the walk
    (each agent's last-token reward) minus the token's value.  Integer-valued operands keep float32 exact."""
    g = torch.Generator().manual_seed(5)
    B, widths = 6, [3, 5, 4]
    vals = [torch.randint(-20, 20, (B, w), generator=g).float() for w in widths]
    rews = [torch.randint(-20, 20, (B, w), generator=g).float() for w in widths]
    gens = [torch.randint(1, w + 1, (B,), generator=g) for w in widths]
    masks = [(torch.arange(w)[None] < n[:, None]).long() for w, n in zip(widths, gens)]
    chains = [(0, 2), (2, 1), (3, 3)]
    adv, ret = OC.marft_gae_unwhitened(rews, vals, masks, chains, 1.0, 1.0)
    for first, n in chains:
        met = 0.0
        for row in range(first, first + n):
            for a in (2, 1, 0):
                n_gen = int(gens[a][row])
                met += float(rews[a][row, n_gen - 1])
                for t in range(n_gen):
                    assert adv[a][row, t] == met - vals[a][row, t]
                    assert ret[a][row, t] == met
                assert not adv[a][row, n_gen:].any()


def _request_batch(mask_dtype=torch.int64):
    r, v, m = _hand_case(mask_dtype)
    batch = {"agent_group_0_token_level_rewards": r[0] * 4, "agent_group_0_values": v[0] * 4,
             "agent_group_0_response_mask": m[0], "token_level_rewards": r[1] * 4, "values": v[1] * 4,
             "response_mask": m[1]}
    extra = {"request_id": np.array(["q", "q"], dtype=object), "traj_len": np.array([2, 2])}
    return SimpleNamespace(batch=batch, non_tensor_batch=extra)


def test_bookkeeping_of_the_full_function():
    data = _request_batch()
    ids = [0]
    assert OC.compute_marft_gae_advantage_return(data, ids, 0.5, 0.5) is None
    assert ids == [0, 1]  # the caller's list grows (reference :395)
    b = data.batch
    assert sorted(k for k in b if k.endswith(("advantages", "returns"))) == [
        "advantages", "agent_group_0_advantages", "agent_group_0_returns", "returns"]
    # four times the hand case: returns are the integer parts, in the mask's dtype
    assert b["returns"].dtype == torch.int64
    assert b["returns"].tolist() == [[20, 64, 0], [27, 77, 293]]
    assert b["agent_group_0_returns"].tolist() == [[141, 0], [25, 54]]
    # advantages: whitened integer parts (float32): mean 0 and unbiased variance 1 over the mask
    raw = torch.tensor([[-12.0, 48.0, 0.0], [-36.0, 45.0, 277.0]])
    sel = raw[data.batch["response_mask"].bool()].numpy().astype(np.float64)
    want = (raw.numpy() - sel.mean()) / np.sqrt(sel.var(ddof=1) + 1e-8)
    assert b["advantages"].dtype == torch.float32
    np.testing.assert_allclose(b["advantages"].numpy(), want, rtol=1e-5, atol=1e-6)


def test_three_agents_store_everything_under_the_last_given_id():
    g = torch.Generator().manual_seed(9)
    B = 4
    batch = {}
    for name, w in (("agent_group_0_", 3), ("agent_group_1_", 2), ("", 4)):
        batch[name + "token_level_rewards"] = torch.randint(-50, 50, (B, w), generator=g).float()
        batch[name + "values"] = torch.randint(-50, 50, (B, w), generator=g).float()
        batch[name + "response_mask"] = torch.ones(B, w, dtype=torch.int64)
    data = SimpleNamespace(batch=batch, non_tensor_batch={"request_id": ["a", "a", "b", "b"], "traj_len": [2, 2, 2, 2]})
    ids = [0, 1]
    OC.compute_marft_gae_advantage_return(data, ids, 1.0, 1.0)
    assert ids == [0, 1, 2]
    assert "agent_group_0_advantages" not in batch and "agent_group_0_returns" not in batch
    adv, ret = OC.marft_gae_unwhitened(
        [batch[n + "token_level_rewards"] for n in ("agent_group_0_", "agent_group_1_", "")],
        [batch[n + "values"] for n in ("agent_group_0_", "agent_group_1_", "")],
        [batch[n + "response_mask"] for n in ("agent_group_0_", "agent_group_1_", "")], [(0, 2), (2, 2)], 1.0, 1.0)
    assert torch.equal(batch["agent_group_1_returns"], ret[1]) and torch.equal(batch["returns"], ret[2])


def test_errors_of_the_reference():
    data = _request_batch()
    with pytest.raises(IndexError):
        OC.compute_marft_gae_advantage_return(data, [], 0.5, 0.5)  # pre_agent_group_ids[-1] of an empty list
    with pytest.raises(KeyError):
        OC.compute_marft_gae_advantage_return(data, [0, 1], 0.5, 0.5)  # no tensors of agent group 1
    with pytest.raises(TypeError):  # range() of a float row sum
        OC.compute_marft_gae_advantage_return(_request_batch(torch.float32), [0], 0.5, 0.5)
    one = _request_batch()
    one.batch["agent_group_0_response_mask"] = torch.tensor([[1, 0], [0, 0]])
    with pytest.raises(ValueError, match="sum of the mask is one"):
        OC.compute_marft_gae_advantage_return(one, [0], 0.5, 0.5)
