import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X and the built HIP kernels")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def tiny_folders(tmp_path_factory):
    """Model folders of the two tiny configurations, written once per session."""
    from helpers import TINY_A, TINY_B, write_tiny
    base = tmp_path_factory.mktemp("models")
    return {"A": write_tiny(base / "A", TINY_A, seed=0), "B": write_tiny(base / "B", TINY_B, seed=1)}
