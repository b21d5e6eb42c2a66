import os
import sys

import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
for p in (ROOT, HERE):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def plain_backend():
    """Run the engine's bookkeeping on the CPU with the plain twins of the kernels."""
    import kernel_twins
    from mini_engine_amd.kernels import ops

    ops.set_backend(kernel_twins.PlainBackend())
    yield
    ops.set_backend(None)


@pytest.fixture(scope="session")
def folders(tmp_path_factory):
    """Model folders with random weights, made once per session in a temporary place."""
    import helpers

    made = {}

    def get(name: str, store_dtype=torch.bfloat16):
        key = (name, store_dtype)
        if key not in made:
            made[key] = helpers.make_folder(name, str(tmp_path_factory.mktemp(f"model_{name}")), store_dtype)
        return made[key]

    return get
