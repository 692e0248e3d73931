import os
import sys

import pytest

ROOT = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


# With DELIVERANCE_SIMT=1 the GPU tests that drive kernels, parts and trace sessions run on the CPU
# instead: the kernels compiled for the host, every operand of every kernel call between protected
# pages (tests/simt).  tests/test_simt.py starts such runs as child processes.
SIMT = os.environ.get("DELIVERANCE_SIMT") == "1"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "needs_device: a GPU test that cannot run on the simulated kernels")
    # the selection of GPU test cases that tests/test_simt.py runs on the simulated kernels by default: simt_quick, or,
    # where two parameter lists cross, a case marked on both (simt_a and simt_b)
    for m in ("simt_quick", "simt_a", "simt_b"):
        config.addinivalue_line("markers", f"{m}: part of the default selection for the simulated kernels")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped where no GPU is visible, so a plain `pytest tests` passes on a CPU box."""
    if SIMT:
        skip = pytest.mark.skip(reason="needs the device itself (streams, graphs, pinned memory)")
        for item in items:
            if "needs_device" in item.keywords:
                item.add_marker(skip)
        return
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


@pytest.fixture(scope="session", autouse=True)
def _simulated_kernels():
    if not SIMT:
        yield
        return
    from simt import harness
    with harness.Sim().patched(auto_guard=True):
        yield


@pytest.fixture(scope="session")
def model_a(tmp_path_factory):
    import helpers
    return helpers.make_model(tmp_path_factory.mktemp("tiny_a"), helpers.CONFIG_A, seed=0)


@pytest.fixture(scope="session")
def model_b(tmp_path_factory):
    import helpers
    return helpers.make_model(tmp_path_factory.mktemp("tiny_b"), helpers.CONFIG_B, seed=1)


@pytest.fixture(scope="session")
def model_a32(tmp_path_factory):
    """Configuration A stored in 32-bit, as openai-community/gpt2 ships."""
    import helpers
    return helpers.make_model(tmp_path_factory.mktemp("tiny_a32"), helpers.CONFIG_A, seed=2, store_dtype="float32")


@pytest.fixture(scope="session")
def model_b32(tmp_path_factory):
    """Configuration B stored in 32-bit, with a head of its own (``tie_word_embeddings`` false)."""
    import helpers
    cfg = dict(helpers.CONFIG_B, tie_word_embeddings=False)
    return helpers.make_model(tmp_path_factory.mktemp("tiny_b32"), cfg, seed=3, store_dtype="float32")


@pytest.fixture(scope="session")
def models(model_a, model_b, model_a32, model_b32):
    return {"A": model_a, "B": model_b, "A32": model_a32, "B32": model_b32}
