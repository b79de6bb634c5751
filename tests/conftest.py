import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from tests import oracle_lib
    return oracle_lib.load()


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def no_handshake_wait_gave_up(request):
    """After every GPU test: no kernel of the library may have given up a handshake wait (the failure record
    of include/hipdma/base.hpp, read through cudadma_device_status).  The one test that provokes it clears
    the record itself."""
    yield
    if request.node.get_closest_marker("gpu") is None:
        return
    import torch
    if not torch.cuda.is_available():
        return
    import cudadma_amd as cd
    bits, waves = cd.device_status(clear=True)
    assert (bits, waves) == (0, 0), f"a handshake wait gave up in {waves} wavefront(s): the results of this test are void"
