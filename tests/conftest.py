import os
import sys

import pytest

ROOT = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped where no GPU is visible, so a plain `pytest tests` passes on a CPU box."""
    try:
        import torch
        have = torch.cuda.is_available()
    except Exception:
        have = False
    if have:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_a(tmp_path_factory):
    import helpers
    return helpers.make_model(tmp_path_factory.mktemp("tiny_a"), helpers.CONFIG_A, seed=0)


@pytest.fixture(scope="session")
def model_b(tmp_path_factory):
    import helpers
    return helpers.make_model(tmp_path_factory.mktemp("tiny_b"), helpers.CONFIG_B, seed=1)


@pytest.fixture(scope="session")
def models(model_a, model_b):
    return {"A": model_a, "B": model_b}
