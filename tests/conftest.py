import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_port():
    import oracle
    if oracle.port is None:
        oracle.build(with_ref=False)
        import importlib
        importlib.reload(oracle)
    return oracle.port


@pytest.fixture(scope="session")
def oracle(oracle_port):
    """The checker package itself (for its float64() switch)."""
    import oracle
    return oracle


@pytest.fixture(scope="session")
def oracle_ref():
    import oracle
    if oracle.ref is None:
        pytest.skip("oracle/_ref (the reference's own CPU build) is not present")
    return oracle.ref
