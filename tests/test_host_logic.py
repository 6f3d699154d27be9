"""Host-side logic of the Python mirror (CPU only): registries, error behaviour, the row-block splitter, the
absence of any CPU fallback."""

from types import SimpleNamespace

import numpy as np
import pytest
import torch


def test_registries_mirror_the_reference():
    import siirl_amd.core_algos as CA

    # every name the reference registers (core_algos.py:572,710,795,865,898,998,1074)
    assert set(CA.POLICY_LOSS_REGISTRY) == {"vanilla", "gspo", "cpgd", "gpg", "clip_cov", "kl_cov", "geo_mean"}
    with pytest.raises(ValueError, match=r"Unsupported loss mode: reinforce. Supported modes are: \["):
        CA.get_policy_loss_fn("reinforce")

    @CA.register_policy_loss("mine")
    def mine(*a, **k):
        return 1

    assert CA.get_policy_loss_fn("mine") is mine
    del CA.POLICY_LOSS_REGISTRY["mine"]

    def est(*a, **k):
        return 2

    CA.register_adv_est("my_est")(est)
    CA.register_adv_est("my_est")(est)  # same function again: allowed
    with pytest.raises(ValueError, match="already been registered"):
        CA.register_adv_est("my_est")(lambda: 3)
    assert CA.get_adv_estimator_fn("my_est") is est
    del CA.ADV_ESTIMATOR_REGISTRY["my_est"]
    assert CA.get_adv_estimator_fn(CA.AdvantageEstimator.GRPO) is CA.compute_grpo_outcome_advantage
    assert CA.AdvantageEstimator.GRPO.value == "grpo" and CA.AdvantageEstimator("gae_marft") is CA.AdvantageEstimator.GAE_MARFT


def test_errors_raised_before_any_device_work():
    import siirl_amd.core_algos as CA

    z = torch.zeros(2, 3)
    with pytest.raises(ValueError, match="Invalid loss_agg_mode: sum"):
        CA.agg_loss(z, z, "sum")
    for bad in ("full", "k3+", "x"):
        with pytest.raises(NotImplementedError):
            CA.kl_penalty(z, z, bad)
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=None, clip_ratio_high=None, clip_ratio_c=1.0)
    with pytest.raises(AssertionError, match="clip_ratio_c"):
        CA.compute_policy_loss_vanilla(z, z, z, z, config=cfg)
    with pytest.raises(AssertionError):
        CA.compute_policy_loss_gspo(z, z, z, z, config=None)
    with pytest.raises(AssertionError):
        CA.get_kl_controller(SimpleNamespace(type="adaptive", kl_coef=0.1, target_kl=0.1, horizon=0))


def test_no_cpu_fallback():
    import siirl_amd.core_algos as CA
    import siirl_amd.torch_functional as SF

    z = torch.zeros(2, 8)
    cfg = SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.2, clip_ratio_c=3.0)
    with pytest.raises(RuntimeError, match="GPU only"):
        SF.logprobs_from_logits(z, torch.zeros(2, dtype=torch.long))
    with pytest.raises(RuntimeError, match="GPU only"):
        SF.entropy_from_logits(z)
    with pytest.raises(RuntimeError, match="GPU only"):
        SF.masked_mean(z, z)
    with pytest.raises(RuntimeError, match="GPU only"):
        CA.agg_loss(z, z, "token-mean")
    with pytest.raises(RuntimeError, match="GPU only"):
        CA.compute_policy_loss_vanilla(z, z, z, z, config=cfg)
    with pytest.raises(RuntimeError, match="GPU only"):
        CA.kl_penalty(z, z, "kl")
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="no GPU"):
            CA.compute_grpo_outcome_advantage(z, z, np.zeros(2, dtype=np.int64))
    with pytest.raises(TypeError):
        SF.logprobs_from_logits(z.long(), torch.zeros(2, dtype=torch.long))


def test_row_blocks():
    from siirl_amd.ops import row_blocks

    x = torch.zeros(6, 10)
    assert list(row_blocks(x)) == [(0, 6, 10)]
    assert list(row_blocks(x[:, :7])) == [(0, 6, 10)]  # row-strided view: one block with stride 10
    y = torch.zeros(3, 5, 10)
    assert list(row_blocks(y)) == [(0, 15, 10)]  # contiguous: collapses
    assert list(row_blocks(y[:, 1:4, :])) == [(0, 3, 10), (50, 3, 10), (100, 3, 10)]  # the actor's response slice
    # (offsets are in elements from the view's own data pointer)
    assert list(row_blocks(torch.zeros(10))) == [(0, 1, 10)]
    assert list(row_blocks(y[:, :, 2:9])) == [(0, 15, 10)]
    with pytest.raises(ValueError):
        list(row_blocks(x.t()))
    w = torch.zeros(2, 3, 4, 10)
    assert list(row_blocks(w[:, :, 1:3, :])) == [(120 * a + 40 * b, 2, 10) for a in range(2) for b in range(3)]


def _views(seed):
    """Random (..., V) views with unit inner stride: slices, steps, size-1 and size-0 axes, expanded leading axes."""
    import random

    rnd = random.Random(seed)
    nd = rnd.randint(1, 4)
    shape = [rnd.choice((0, 1, 2, 3, 5)) if rnd.random() < 0.9 else 1 for _ in range(nd - 1)] + [rnd.choice((1, 4, 9))]
    base = torch.zeros(shape)
    v = base
    for d in range(nd):
        n = v.shape[d]
        if n >= 2 and rnd.random() < 0.6:
            lo = rnd.randint(0, n - 1)
            hi = rnd.randint(lo + 1, n)
            step = rnd.choice((1, 1, 2)) if d < nd - 1 else 1
            v = v[(slice(None),) * d + (slice(lo, hi, step),)]
    if nd >= 2 and rnd.random() < 0.2:
        v = v.unsqueeze(0)
    return v


def test_cpp_row_blocks_agree_with_the_python_statement():
    """The C++ layer cuts a logits view into uniformly strided row blocks before it launches anything; an error there
    would send a kernel to memory the view does not own.  Same answer as the Python statement of the rule on 2000
    random views, and every block stays inside the view's storage."""
    from siirl_amd.ops import row_blocks

    for seed in range(2000):
        v = _views(seed)
        want = [t for blk in row_blocks(v) if blk[1] for t in blk]
        got = list(torch.ops.siirl_hip.row_blocks(v))
        got = [t for i in range(0, len(got), 3) if got[i + 1] for t in got[i:i + 3]]
        assert got == want, (seed, tuple(v.shape), v.stride(), got, want)
        V = v.shape[-1]
        limit = v.untyped_storage().nbytes() // v.element_size() - v.storage_offset()
        rows = 0
        for i in range(0, len(got), 3):
            off, n, stride = got[i:i + 3]
            assert off >= 0 and off + (n - 1) * stride + V <= limit
            rows += n
        assert rows == (v.numel() // V if V else 0)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_response_window_helpers_refuse_the_cpu_and_bad_arguments():
    """The helpers of siirl/utils/model_utils/torch_functional.py:209-254,416-500,638-647: CPU tensors raise (no CPU
    fallback), argument errors surface before any device work; remove_pad_token is host-side list building."""
    import siirl_amd.fused_linear as FL
    import siirl_amd.torch_functional as SF
    from oracle import padding as OP

    ids = torch.tensor([[5, 1, 0, 0], [7, 8, 9, 1]])
    with pytest.raises(RuntimeError, match="GPU only"):
        SF.get_response_mask(ids, 1)
    with pytest.raises(RuntimeError, match="GPU only"):
        SF.get_eos_mask(ids, 1)
    with pytest.raises(RuntimeError):
        SF.get_unpad_data(torch.ones(2, 4, dtype=torch.long))
    with pytest.raises(RuntimeError, match="GPU only"):
        SF.log_probs_from_logits_response(ids, torch.zeros(2, 4, 11), 2)
    mask = torch.tensor([[0, 0, 1, 1], [1, 1, 1, 1]])
    assert SF.remove_pad_token(ids, mask) == OP.remove_pad_token(ids.numpy(), mask.numpy()) == [[0, 0], [7, 8, 9, 1]]
    with pytest.raises(RuntimeError, match="GPU only"):
        FL.fused_linear_logprob_entropy(torch.zeros(2, 64, dtype=torch.bfloat16), torch.zeros(9, 64, dtype=torch.bfloat16),
                                        torch.zeros(2, dtype=torch.long))
    with pytest.raises(ValueError):
        FL.set_saved_logits_limit(-5)


def test_uid_codes_for_keys_that_are_not_int64():
    """Host side of the group operators: uids the reference would use as dict keys (core_algos.py:326,
    filter_interface/dapo.py:70) become int64 codes with the same equalities."""
    import numpy as np
    import torch

    from siirl_amd import core_algos as CA
    from siirl_amd import dapo_filter as DF

    big = [2 ** 100 + 3, 5, 2 ** 100 + 3, -7, 5]
    want = [0, 1, 0, 2, 1]
    assert CA._uid_tensor(big, 5, "cpu").tolist() == want
    assert CA._uid_tensor(np.asarray(big, dtype=object), 5, "cpu").tolist() == want
    assert CA._uid_tensor(["10", "2", "10", "3", "2"], 5, "cpu").tolist() == want  # int() per entry, as the reference
    assert CA._uid_tensor(np.asarray([2 ** 63 + 1, 4, 2 ** 63 + 1], dtype=np.uint64), 3, "cpu").tolist() == [0, 1, 0]
    assert CA._uid_tensor(np.asarray([9, -4, 9]), 3, "cpu").tolist() == [9, -4, 9]  # integer arrays pass through
    assert CA._uid_tensor(torch.tensor([9, -4, 9]), 3, "cpu").tolist() == [9, -4, 9]
    with pytest.raises(ValueError):
        CA._uid_tensor(["a", "b"], 2, "cpu")  # the reference's int("a")
    with pytest.raises(ValueError):
        CA._uid_tensor([1, 2, 3], 2, "cpu")
    assert DF._uid_tensor(["a", "b", "a", "c"], "cpu").tolist() == [0, 1, 0, 2]  # the filter keys Python objects as is
    assert DF._uid_tensor(big, "cpu").tolist() == want
    assert DF._uid_tensor(np.asarray([3, 3, 1]), "cpu").tolist() == [3, 3, 1]
    with pytest.raises(ValueError):
        DF._uid_tensor(np.asarray(["a", "b"]), "cpu")  # numpy strings have .item: int() as in the reference


def test_marft_requests_must_not_overlap():
    """Requests whose row ranges overlap are refused on the host, before anything is launched (the reference walks
    them sequentially, last writer wins; concurrent waves would race); ranges that touch are fine."""
    from siirl_amd.core_algos import _check_marft_chains

    _check_marft_chains([(0, 4), (4, 4), (8, 2)], 10)
    _check_marft_chains([(4, 4), (0, 4)], 8)  # any order
    _check_marft_chains([], 0)
    with pytest.raises(NotImplementedError, match="runs into"):
        _check_marft_chains([(0, 5), (4, 4)], 10)
    with pytest.raises(NotImplementedError, match="runs into"):
        _check_marft_chains([(4, 4), (0, 6)], 10)
    with pytest.raises(IndexError):
        _check_marft_chains([(0, 4), (4, 7)], 10)
