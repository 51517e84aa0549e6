import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """The tests load the in-tree library and call it only; a tree where nothing is built yet gets built once."""
    from turboexl3_amd import _lib, build

    if not os.path.exists(_lib.LIB_PATH):
        build.build()


def has_gpu() -> bool:
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o

    o.build()
    return o


@pytest.fixture(autouse=True)
def workspace_head_stays_zero(request):
    """The C ABI's workspace contract: the first T3_WORKSPACE_COUNTER_BYTES bytes (the fused launches' arrival counters)
    are zero when a workspace is first passed and every call leaves them zero, whichever entry points share it. The
    harness keeps one workspace a device; after every GPU test its head must still be zero."""
    yield
    if request.node.get_closest_marker("gpu") is None:
        return
    api = sys.modules.get("turboexl3_amd.api")
    if api is None:
        return
    for ws in api._workspaces.values():
        assert not ws[:65536].any().item(), "a call left the workspace's counter area nonzero"
