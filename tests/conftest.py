import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)                                    # `oracle` package (test infrastructure)
sys.path.insert(0, os.path.join(ROOT, "history-cache_amd"))  # `hiscache`, `hiscache_backend`


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    from oracle import hc_oracle
    hc_oracle.build()
    return hc_oracle
