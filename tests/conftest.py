import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (MI355X); run with -m gpu")


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def balanced_schedule_for_small_shapes(monkeypatch):
    """The GPU tests run small shapes with partition_size = 0 to exercise the balanced decode
    schedule; without this the library would route such calls to the grid schedule (its choice
    for latency-bound calls).  Tests of that choice delete the variable again."""
    monkeypatch.setenv("AICOMP_KV_SMALL_DECODE_TOKENS", "0")
