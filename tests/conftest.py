"""Shared pytest configuration: the `gpu` marker and import paths."""

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def ct():
    import causal_trainer_dev_amd

    return causal_trainer_dev_amd


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    import causal_trainer_dev_amd

    causal_trainer_dev_amd._lib.load()  # fail loudly if the HIP library is missing
    return torch.device("cuda:0")
