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


def pytest_terminal_summary(terminalreporter):
    """The observed attention errors of this run, worst comparison per test (the caps are in helpers.py)."""
    try:
        import helpers
    except ImportError:
        return
    if not helpers.OBSERVED:
        return
    worst = {}
    for test, what, max_abs, rel, numel in helpers.OBSERVED:
        w = worst.setdefault(test, [0.0, 0.0, 0])
        w[0], w[1], w[2] = max(w[0], max_abs), max(w[1], rel), w[2] + 1
    tr = terminalreporter
    tr.write_sep("-", f"observed attention error vs the fp32 oracle (caps: max abs {helpers.ATTN_MAX_ABS}, relative {helpers.ATTN_MAX_REL})")
    for test, (a, r, n) in sorted(worst.items()):
        tr.write_line(f"{a:.3e}  {r:.3e}  {n:4d} comparisons  {test}")
    tr.write_line(f"overall: max abs {max(w[0] for w in worst.values()):.3e}, relative {max(w[1] for w in worst.values()):.3e}")
