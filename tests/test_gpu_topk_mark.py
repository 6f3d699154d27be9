"""``siirl_topk_mark`` (the selection step of KL-Cov, reference ``siirl/dag_worker/core_algos.py:1055-1063``) against
a sort on the host.  Index work: the marked set must be exactly the k largest scores, ties at the cut resolved towards
the lowest index; bit-exact, no tolerance."""
import numpy as np
import pytest
import torch

import siirl_amd.ops  # noqa: F401  (loads torch.ops.siirl_hip.*)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _expected(scores: np.ndarray, k: int) -> np.ndarray:
    """Indices of the k largest, NaN above everything, -0 == +0, ties towards the lowest index (a stable sort of the
    negated scores)."""
    s = scores.astype(np.float64)
    s = np.where(np.isnan(s), np.inf, s)
    rank = np.where(np.isnan(scores), 2.0, np.where(np.isposinf(scores), 1.0, 0.0))  # NaN above +inf
    order = np.lexsort((np.arange(len(s)), -s, -rank))  # last key is the primary one
    return np.sort(order[:k])


def _run(scores: torch.Tensor, k: int, value=0.75):
    marks = torch.ops.siirl_hip.topk_mark(scores.to(DEV), k, value)
    assert marks.shape == scores.shape and marks.dtype == torch.float32
    m = marks.cpu().numpy().reshape(-1)
    assert set(np.unique(m)) <= {0.0, np.float32(value)}
    return np.nonzero(m)[0]


@pytest.mark.parametrize("n", [1, 2, 3, 5, 63, 64, 1000, 4096, 4097, 100_003, 1_048_576 + 7])
def test_random_scores(n):
    g = torch.Generator().manual_seed(n)
    x = torch.randn(n, generator=g) * torch.exp(torch.randn(n, generator=g))
    for k in sorted({0, 1, 2, max(1, n // 5000), n // 7, n - 1, n}):
        if 0 <= k <= n:
            assert np.array_equal(_run(x, k), _expected(x.numpy(), k)), (n, k)


def test_heavy_ties_and_special_values():
    g = torch.Generator().manual_seed(5)
    n = 300_000
    x = torch.randint(-3, 4, (n,), generator=g).float()  # seven distinct values: every cut falls inside a tie
    for k in (1, 17, 40_000, 150_000, 299_999):
        assert np.array_equal(_run(x, k), _expected(x.numpy(), k)), k
    const = torch.zeros(50_000)
    const[::2] = -0.0  # -0 and +0 are one value
    assert np.array_equal(_run(const, 12_345), np.arange(12_345))
    y = torch.randn(20_000, generator=g)
    y[100], y[7000], y[19_999] = float("nan"), float("inf"), float("nan")
    y[5:50] = float("-inf")
    for k in (1, 2, 3, 4, 19_990, 20_000):
        assert np.array_equal(_run(y, k), _expected(y.numpy(), k)), k
    # the masked tail of a covariance matrix: long stretches of -inf
    z = torch.randn(64, 4096, generator=g)
    lens = torch.randint(1, 4097, (64,), generator=g)
    z[torch.arange(4096)[None, :] >= lens[:, None]] = float("-inf")
    k = int(lens.sum()) // 50
    assert np.array_equal(_run(z, k), _expected(z.numpy().reshape(-1), k))
    k = int(lens.sum()) + 10  # more than the finite entries: the lowest-index -inf entries fill up
    assert np.array_equal(_run(z, k), _expected(z.numpy().reshape(-1), k))


def test_ties_across_several_tiles_of_a_chunk():
    """3 M scores of seven distinct values: a workgroup's chunk spans three tiles, so the rank of an entry at the cut
    runs over tiles and chunks."""
    g = torch.Generator().manual_seed(6)
    n = 3_000_000 + 3
    x = torch.randint(-3, 4, (n,), generator=g).float()
    for k in (5, 430_000, 1_500_000, n - 2):
        assert np.array_equal(_run(x, k), _expected(x.numpy(), k)), k


def test_unaligned_and_refusals():
    g = torch.Generator().manual_seed(9)
    base = torch.randn(10_001, generator=g).to(DEV)
    view = base[1:]  # 4-byte aligned only: the scalar path
    marks = torch.ops.siirl_hip.topk_mark(view.contiguous(), 77, 1.0)
    assert np.array_equal(np.nonzero(marks.cpu().numpy())[0], _expected(view.cpu().numpy(), 77))
    with pytest.raises(RuntimeError):
        torch.ops.siirl_hip.topk_mark(base, 10_002, 1.0)
    with pytest.raises((RuntimeError, ValueError)):
        torch.ops.siirl_hip.topk_mark(base[::2], 3, 1.0)  # not contiguous
    assert torch.ops.siirl_hip.topk_mark(base[:0], 0, 1.0).numel() == 0


def test_at_batch_scale_against_torch_topk():
    """45 M scores (a [5488, 8192] batch): same set as torch.topk where the cut has no tie."""
    g = torch.Generator(device=DEV).manual_seed(1)
    x = torch.randn(5488 * 8192, device=DEV, generator=g)
    k = 4637
    marks = torch.ops.siirl_hip.topk_mark(x, k, 1.0)
    want = torch.zeros_like(x)
    want[torch.topk(x, k).indices] = 1.0
    assert int(marks.sum()) == k and torch.equal(marks, want)


def test_sweep_random_selections():
    """Seeded random sizes, value distributions (continuous, a handful of distinct values, masked -inf stretches, NaN
    sprinkled in) and k; ``SIIRL_TEST_SEED=<int>`` shifts the seeds."""
    import os

    shift = 100003 * int(os.environ.get("SIIRL_TEST_SEED", "0"))
    rng = np.random.default_rng(4242 + shift)
    for case in range(80):
        n = int(rng.choice([1, 2, 7, 64, 65, 4095, 4096, 4097, 20_000, 70_001, 300_000]))
        kind = case % 5
        if kind == 0:
            x = rng.standard_normal(n).astype(np.float32) * np.float32(10.0 ** rng.integers(-3, 4))
        elif kind == 1:
            x = rng.integers(-2, 3, n).astype(np.float32)
        elif kind == 2:
            x = rng.standard_normal(n).astype(np.float32)
            x[rng.random(n) < rng.random()] = -np.inf
        elif kind == 3:
            x = rng.standard_normal(n).astype(np.float32)
            x[rng.random(n) < 0.01] = np.nan
            x[rng.random(n) < 0.01] = np.inf
        else:
            x = np.full(n, np.float32(rng.standard_normal()), dtype=np.float32)
        k = int(rng.integers(0, n + 1)) if case % 3 else int(min(n, max(1, n // 5000)))
        got = _run(torch.from_numpy(x), k)
        assert np.array_equal(got, _expected(x, k)), (case, n, kind, k)


# ------------------------------------------------------------------------------------------ entries inside an interval


@pytest.mark.parametrize("n", [0, 1, 5, 4096, 4097, 250_001, 3_000_003])
def test_range_indices_equals_nonzero(n):
    """``range_indices`` (Clip-Cov's candidate list, reference ``core_algos.py:974-975``) against torch.nonzero of the
    same two comparisons: same indices in the same (ascending) order, bit-exact."""
    g = torch.Generator().manual_seed(n + 1)
    x = torch.randn(n, generator=g) * 2
    if n > 10:
        x[torch.rand(n, generator=g) < 0.3] = float("-inf")
        x[3], x[7] = float("nan"), float("inf")
    xd = x.to(DEV)
    for lo, hi in ((1.0, 5.0), (-0.5, 0.5), (10.0, 20.0), (float("-inf"), float("inf")), (0.0, 0.0)):
        got = torch.ops.siirl_hip.range_indices(xd, lo, hi)
        want = torch.nonzero((x < hi) & (x > lo)).reshape(-1)
        assert got.dtype == torch.int64 and torch.equal(got.cpu(), want), (n, lo, hi, got.numel(), want.numel())
    m = torch.randn(37, 129, generator=g).to(DEV)  # a matrix: flat, row-major indices
    got = torch.ops.siirl_hip.range_indices(m, 0.2, 1.1)
    assert torch.equal(got.cpu(), torch.nonzero(((m < 1.1) & (m > 0.2)).reshape(-1).cpu()).reshape(-1))
