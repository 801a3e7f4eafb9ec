import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "sanitize: CPU sanitizer builds in child processes (compiles for ~30 s)")


@pytest.fixture(scope="session")
def oracle_mod():
    import oracle

    oracle.lib()  # builds the checker if it is missing
    return oracle
