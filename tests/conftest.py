import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a MI355X (run with -m gpu); everything else runs on the CPU")
    # tests read loss scalars with float(); where the scalar still carries a graph torch warns once per process
    config.addinivalue_line("filterwarnings",
                            "ignore:Converting a tensor with requires_grad=True to a scalar:UserWarning")


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _announce(request):
    # name the case before it touches the GPU, so that a fault can be attributed
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield

