import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    config.addinivalue_line("markers", "delegates: in-tree test whose inputs a \"hip\" operator hands to the host operator")


@pytest.fixture(scope="session")
def port():
    from oracle import port as p
    p.lib()
    p.set_threads(min(8, p.max_threads()))
    return p


@pytest.fixture(scope="session")
def ref():
    """The compiled TenniS reference; present only where oracle/_ref was built."""
    from oracle import ref as r
    if not r.available():
        pytest.skip("compiled reference (oracle/_ref) not built in this tree")
    r.lib()
    return r
