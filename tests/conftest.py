import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) GPU and the built HIP extension")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def risa():
    """The product package, with a loud failure when the HIP extension is missing on a GPU box."""
    import torch

    import risaattention_amd

    if torch.cuda.is_available():
        from risaattention_amd import native

        native.library()  # raises when the shared library was not built
        assert risaattention_amd.int8_attention_is_available(), "HIP extension loaded but device is not gfx950"
    return risaattention_amd
