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
    from oracle import oracle as orc
    orc.build()
    return orc


@pytest.fixture(params=["merge-path", "row-blocks"])
def push_aggregation(request, monkeypatch):
    """Which kernels PR_PEVal / PR_IncEVal aggregate with.  The library picks by subgraph size (row blocks from about
    67 M edges); the environment variable moves the limit, so small test graphs can take the large-graph path."""
    if request.param == "row-blocks":
        monkeypatch.setenv("DRONE_PR_ROWBLOCK_MIN_EDGES", "1")
    else:
        monkeypatch.delenv("DRONE_PR_ROWBLOCK_MIN_EDGES", raising=False)
    return request.param
