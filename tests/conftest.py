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


def pytest_terminal_summary(terminalreporter):
    """The plain kernels' bfloat16 errors that this run measured, beside the recorded figures they are held to."""
    import helpers
    if not helpers.MEASURED_PLAIN_BF16_REL:
        return
    terminalreporter.write_line("plain kernels in bfloat16, largest error relative to the largest logit (measured / recorded):")
    for label, rel in sorted(helpers.MEASURED_PLAIN_BF16_REL.items()):
        rec = helpers.PLAIN_BF16_REL.get(label)
        terminalreporter.write_line(f"  {label}: {rel:.3e} / {'-' if rec is None else format(rec, '.3e')}")
