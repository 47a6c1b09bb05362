import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda", 0)


@pytest.fixture(autouse=True)
def _seeded():
    """Every test starts from the same state of torch's default generators (CPU and GPU), so that
    inputs drawn without a generator of their own are the same in every run and a tolerance that
    holds once holds always."""
    import torch
    torch.manual_seed(20240531)
    yield
