import os
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _seed():
    # the reference seeds torch to 0 before every test (tests/conftest.py:11-15)
    torch.manual_seed(0)
    yield


@pytest.fixture(scope="session")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def announce(msg: str) -> None:
    """Names the case before a GPU step, flushed, so a dead box still tells which case ran."""
    print(f"[case] {msg}", flush=True)
