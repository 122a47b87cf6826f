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


@pytest.fixture(params=[("direct", None), ("staged", None), ("staged", 1), ("staged", 3), ("direct", 3)],
                ids=["direct", "window=all", "window=1", "window=3", "direct-window=3"])
def rotation_window(request):
    """Runs a GPU test under the rotation schedules: shards read from their home rows by one grouped launch per
    layer (the default); and, staged through the two HBM slots, all shards of a layer together, one shard per ring
    step (the reference's schedule) and a window that does not divide the shard count (ragged last window); the
    ragged window once more without staging."""
    from rtp_amd.ring import set_rotation_mode, set_rotation_window
    mode, window = request.param
    set_rotation_mode(mode)
    set_rotation_window(window)
    yield window
    set_rotation_window(None)
    set_rotation_mode("direct")
