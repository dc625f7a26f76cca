"""Test configuration: `gpu` marks tests that need a MI355X; everything else runs on the CPU."""

import pathlib
import sys

import numpy as np
import pytest
import torch

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config: pytest.Config) -> None:
    config.addinivalue_line("markers", "gpu: needs a HIP device and the built libmlkit_amd.so")


def pytest_collection_modifyitems(config: pytest.Config, items: list[pytest.Item]) -> None:
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def deterministic_seeds():
    torch.manual_seed(0)
    np.random.seed(0)
    yield


@pytest.fixture
def rng() -> np.random.Generator:
    return np.random.default_rng(1234)
