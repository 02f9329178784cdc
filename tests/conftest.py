import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def cuda():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    # Fails loudly if the HIP library was never built: there is no fallback.
    from iron_amd._lib import lib

    lib()
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _name_the_case(request):
    """Name each GPU case on stderr before it launches, so a fault names its test."""
    if request.node.get_closest_marker("gpu"):
        print(f"[gpu case] {request.node.nodeid}", file=sys.stderr, flush=True)
    yield
