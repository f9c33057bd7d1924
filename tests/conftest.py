import os
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (REPO, os.path.join(REPO, "amd-pace_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _gpu_present() -> bool:
    import torch

    return torch.cuda.is_available()


@pytest.fixture(scope="session")
def device():
    import torch

    if not _gpu_present():
        pytest.skip("no GPU in this environment")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _announce(request):
    # Name the case before it touches the GPU, so that a lost box still tells which test ran.
    if request.node.get_closest_marker("gpu"):
        sys.stdout.write(f"\n[gpu-case] {request.node.nodeid}\n")
        sys.stdout.flush()
    yield
