import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu() -> bool:
    # /dev/kfd is present exactly when an AMD GPU is usable; cheaper than importing torch.
    return os.path.exists("/dev/kfd")


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def goldens():
    import json
    with open(Path(__file__).parent / "golden" / "reference_goldens.json") as f:
        return json.load(f)


@pytest.fixture(scope="session")
def segops_lib():
    from futhark_amd import Segops
    return Segops()


@pytest.fixture(scope="session")
def ctx(segops_lib):
    """One context for the whole GPU session (its free list and scratch get reused)."""
    from futhark_amd import Context
    c = Context(segops_lib)
    yield c
    c.close()
