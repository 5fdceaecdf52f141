import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (gfx950) device")


@pytest.fixture
def recomputing_backward():
    """The split backward without its dS workspace (the dQ kernel recomputes S and dP); the
    library's default limit is restored afterwards."""
    from aotriton_amd._lib import lib
    lib.fa_set_bwd_workspace_limit(0)
    yield
    lib.fa_set_bwd_workspace_limit(-1)
