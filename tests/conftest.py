import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    from oracle import pyoracle
    return pyoracle.oracle()


@pytest.fixture(scope="session")
def ref():
    from oracle import pyoracle
    if not pyoracle.Reference.available():
        pytest.skip("oracle/_ref/libnnacl_ref.so not built (reference tree absent)")
    return pyoracle.reference()
