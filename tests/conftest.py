import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def tiny_graphs():
    """A few hand-sized symmetric CSR graphs with self-loops: (indptr, col) int32 numpy."""
    from tests.helpers import random_symmetric_csr
    return [random_symmetric_csr(n, m, seed) for n, m, seed in
            [(1, 0, 0), (2, 1, 1), (7, 9, 2), (33, 80, 3), (64, 400, 4), (130, 260, 5)]]
