import os

# the parity tests exercise the built-in heuristics: the shipped tuning table is loaded only where a test asks for it
os.environ.setdefault("SGEMM_TUNING_TABLE", "none")
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as orc
    return orc
