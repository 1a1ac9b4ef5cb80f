import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def engine_factory():
    """Creates engines on cuda:0 and closes them at session end."""
    made = []

    def make(num_vranks):
        from pccl_amd.engine import Engine
        e = Engine(num_vranks, 0)
        made.append(e)
        return e

    yield make
    for e in made:
        e.close()
