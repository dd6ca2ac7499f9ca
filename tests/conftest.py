import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders of the tiny configurations, written once per session into a temporary folder."""
    import helpers
    base = tmp_path_factory.mktemp("models")
    return helpers.ModelDirs(str(base))


@pytest.fixture(scope="session")
def bf16_bound():
    """The tolerance of bfloat16 engines with tuned kernels: see helpers.Bf16Bound."""
    import helpers
    return helpers.Bf16Bound()
