"""Shared fixtures.  GPU tests are marked `gpu`; everything else runs on the CPU."""
import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def orc():
    from oracle import pyoracle
    pyoracle.build()
    return pyoracle


@pytest.fixture()
def rng():
    return np.random.default_rng(20240611)


@pytest.fixture()
def hooked():
    """The test flavour of the kernel library (libag_hip_test.so: the same sources built with the tuning hooks of
    csrc/ag_test_hooks.h) for the duration of one test: every launcher of kernels.py goes through it, and the test
    can force tile configurations, split counts and chunk sizes.  The shipped library has no such hooks."""
    from __graft_entry__ import load_package

    load_package()
    from rust_autograd_amd import capi

    with capi.use_test_library() as lib:
        yield lib
