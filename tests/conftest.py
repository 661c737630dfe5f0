import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    """The C restatement of the reference kernels (the checker)."""
    import oracle
    return oracle.require_ops()


@pytest.fixture(scope="session")
def ref():
    """The reference's own kernels compiled in place, when that build is present."""
    import oracle
    if oracle.ref is None:
        pytest.skip("oracle/_ref not built (needs the reference checkout at build time)")
    return oracle.ref
