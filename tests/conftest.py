import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
TESTS = os.path.dirname(os.path.abspath(__file__))
if TESTS not in sys.path:
    sys.path.insert(0, TESTS)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """Model folders of the tiny configurations, written once per session into a
    temporary place by the framework's random-weights mode."""
    from helpers import TINY, write_tiny
    root = tmp_path_factory.mktemp("models")
    return {name: write_tiny(name, str(root / name)) for name in TINY}


@pytest.fixture(scope="session")
def varied_folders(tmp_path_factory):
    """Model folders of the configurations whose greedy continuation varies."""
    from helpers import VARIED, write_tiny
    root = tmp_path_factory.mktemp("varied_models")
    return {name: write_tiny(name, str(root / name)) for name in VARIED}
