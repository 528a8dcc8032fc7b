import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    from checkers import Checker
    return Checker("orc")


@pytest.fixture(scope="session")
def ref():
    from checkers import Checker, have_ref
    if not have_ref():
        pytest.skip("oracle/_ref/libmshadow_ref.so not built (needs /root/reference)")
    return Checker("ref")
