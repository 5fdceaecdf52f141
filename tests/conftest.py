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


@pytest.fixture(params=['workspace', 'no workspace'])
def with_and_without_workspace(request):
    """Runs a test twice: with the library's workspace (packed copies of tensors whose rows are not
    made of aligned 16-byte pieces reach the MFMA kernels; dS kept in HBM) and with the limit at 0
    (element-wise vector-ALU kernels; recomputing backward)."""
    from aotriton_amd._lib import lib
    lib.fa_set_bwd_workspace_limit(-1 if request.param == 'workspace' else 0)
    yield request.param
    lib.fa_set_bwd_workspace_limit(-1)
