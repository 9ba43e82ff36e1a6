import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _library_default_store_policy(request):
    """Tests set the library's process-wide store-policy options: every GPU test starts from the library's own
    defaults, whatever the test before it chose."""
    if "gpu" in request.keywords:
        from yafsdp_amd import _native

        _native.set_store_policy("rotating_sets")
    yield
