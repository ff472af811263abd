import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "appmult-aware-retraining_amd")
GOLDEN = os.path.join(ROOT, "tests", "golden")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN


@pytest.fixture(scope="session")
def oracle():
    from oracle import lutgemm_oracle as O
    O.build_c_oracle()
    return O


@pytest.fixture(autouse=True)
def _seed_per_test(request):
    """Every test draws its torch random numbers from a seed of its own name: the same data whether the test runs alone,
    in another order or after other tests (tests that seed a generator themselves are not affected)."""
    import zlib
    try:
        import torch
    except ImportError:
        yield
        return
    torch.manual_seed(zlib.crc32(request.node.nodeid.encode()))
    yield
