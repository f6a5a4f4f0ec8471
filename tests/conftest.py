import importlib
import os
import sys

import pytest

# Tests name the route they mean to exercise: the one-time timing of both routes for many rows of x
# (functional._measure_route) stays off unless a test switches it on.
os.environ.setdefault("NF4HIP_CALIBRATE", "0")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TESTS = os.path.dirname(os.path.abspath(__file__))
if TESTS not in sys.path:
    sys.path.insert(0, TESTS)
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ta():
    """The package under test (its directory name is not a Python identifier)."""
    return importlib.import_module("lightning-thunder_amd")


@pytest.fixture(scope="session")
def oracle():
    from oracle import nf4_oracle

    nf4_oracle.C()  # build/load the C checker once
    return nf4_oracle
