import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def rel_l2(actual, expected):
    actual, expected = actual.double().cpu(), expected.double().cpu()
    return ((actual - expected).norm() / expected.norm().clamp_min(1e-30)).item()


@pytest.fixture(scope="session")
def golden_dir():
    return ROOT / "tests" / "golden"
