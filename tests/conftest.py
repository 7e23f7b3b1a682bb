import os
import sys

import pytest

# Tests that read generated source or count compilations must see every graph lowered, also on a
# machine whose Inductor disk cache already holds it from an earlier run.
os.environ.setdefault("TORCHINDUCTOR_FORCE_DISABLE_CACHES", "1")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
