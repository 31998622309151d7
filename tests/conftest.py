import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) GPU")


def pytest_collection_modifyitems(config, items):
    # announce every GPU case before it runs so that a lost box still names the case
    pass


@pytest.fixture(autouse=True)
def _announce(request):
    if request.node.get_closest_marker("gpu") is not None:
        print(f"\n[gpu-case] {request.node.nodeid}", flush=True)
    yield


def bf16_np(t):
    """torch bf16/fp16 tensor -> fp32 numpy (exact)."""
    return t.detach().float().cpu().numpy()


def words_np(t):
    """int64 mask tensor -> uint64 numpy."""
    return t.detach().cpu().numpy().view(np.uint64)
