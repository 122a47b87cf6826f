import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950); run with -m gpu on the GPU box")


@pytest.fixture(autouse=True)
def _seed():
    import torch

    torch.manual_seed(0)
    yield


@pytest.fixture(params=[None, 1, 3], ids=["window=all", "window=1", "window=3"])
def rotation_window(request):
    """Runs a GPU test under three rotation schedules: all shards of a layer staged together (one grouped
    launch per layer), one shard per ring step (the reference's schedule), and a window that does not
    divide the shard count (ragged last window)."""
    from rtp_amd.ring import set_rotation_window
    set_rotation_window(request.param)
    yield request.param
    set_rotation_window(None)
