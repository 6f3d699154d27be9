"""GPU parity: the per-step data metrics (through the C ABI) vs the CPU oracle.  Counts, lengths, clip ratios and
the max / min of tensor elements exact; means, the statistics of the per-sequence score / reward sums (sums of up
to L float32 terms) and the explained variance within 1e-5 relative (+1e-6)."""
import pytest
import torch

from oracle import metric_utils as OM
from test_oracle_metrics import make_data

pytestmark = pytest.mark.gpu

EXACT = ("max", "min", "clip_ratio/mean")


def _compare(got, want):
    for k, w in want.items():
        g = got[k]
        if (k.endswith(EXACT) and "score" not in k and "rewards" not in k) or ("length" in k and not k.endswith("mean")):
            assert g == w, (k, g, w)
        else:
            assert abs(g - w) <= 1e-6 + 1e-5 * abs(w), (k, g, w)


@pytest.mark.parametrize("B,P,L", [(2, 1, 1), (16, 7, 33), (64, 100, 5000), (300, 20, 4096)])
@pytest.mark.parametrize("with_values", [True, False])
@pytest.mark.parametrize("on_gpu", [True, False])
def test_compute_data_metric(dev, B, P, L, with_values, on_gpu):
    from siirl_amd.metric_utils import compute_data_metric

    data = make_data(B, P, L, B + L, with_values)
    want = OM.compute_data_metric(data)
    inp = {k: (v.to(dev) if on_gpu else v) for k, v in data.items()}
    got = compute_data_metric(inp)
    assert set(want) <= set(got)
    _compare(got, want)
    assert ("critic/values/mean" in got) == with_values


def test_mask_dtypes_and_all_wrong(dev):
    from siirl_amd.metric_utils import compute_data_metric

    data = make_data(8, 4, 17, 3)
    data["token_level_rewards"] = torch.zeros(8, 17)  # nobody is "correct": those three entries are 0
    data["token_level_scores"] = torch.zeros(8, 17)
    want = OM.compute_data_metric(data)
    for dt in (torch.bool, torch.int32, torch.float32):
        inp = {k: v.to(dev) for k, v in data.items()}
        inp["response_mask"] = inp["response_mask"].to(dt)
        inp["attention_mask"] = inp["attention_mask"].to(dt)
        got = compute_data_metric(inp)
        _compare(got, want)
        assert got["response/correct_length/max"] == 0 and got["response/correct_length/mean"] == 0
    import numpy as np

    inp["__num_turns__"] = np.array([1, 2, 3, 2, 1, 1, 1, 5])
    got = compute_data_metric(inp)
    assert int(got["num_turns/max"]) == 5 and "perf/process_cpu_mem_used_gb" in got
