import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN


@pytest.fixture(autouse=True)
def _poisoned_allocator(request):
    """Before every GPU test, memory that torch's caching allocator will hand out next is filled with 0xFF bytes (NaN in
    bf16, fp16, fp32 and e4m3fn; -NaN-like garbage in e5m2), so that a kernel which reads bytes nobody wrote -- padding of
    a k-blocked copy, a workspace expected to be zero, the tail of a ragged row -- shows up in the comparison instead of
    passing on the zero pages a fresh process happens to get."""
    if request.node.get_closest_marker("gpu") is None:
        yield
        return
    import torch

    if torch.cuda.is_available():
        big = torch.full((256 << 20,), 0xFF, dtype=torch.uint8, device="cuda")       # the allocator's pool of large blocks
        small = [torch.full((256 << 10,), 0xFF, dtype=torch.uint8, device="cuda") for _ in range(64)]  # and of small ones
        del big, small
    yield
