import importlib
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def oracle():
    return importlib.import_module("oracle.moe_i8_oracle")


@pytest.fixture
def pra():
    """The product package (directory ``prime-rl_amd``) through its import alias."""
    return importlib.import_module("prime_rl_amd")


@pytest.fixture
def gen():
    return torch.Generator(device="cpu").manual_seed(1234)


@pytest.fixture(scope="session")
def golden():
    import json

    with open(ROOT / "tests" / "golden" / "known_answers.json") as f:
        return json.load(f)
