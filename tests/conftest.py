"""Shared pytest configuration.

`-m "not gpu"` covers the CPU oracle against golden vectors and known answers,
the host-side logic and the loadability of the C-ABI library.  `-m gpu` tests
are the parity tests proper: they call the HIP kernels through the C ABI on a
real MI355X and compare with the oracle.
"""
import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
TESTS = os.path.dirname(os.path.abspath(__file__))
if TESTS not in sys.path:
    sys.path.insert(0, TESTS)


def pytest_configure(config):
    config.addinivalue_line(
        "markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.binding import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def reference():
    """The compiled reference CPU backend, where oracle/_ref was built."""
    from oracle.binding import Reference
    if not Reference.available():
        pytest.skip("oracle/_ref/libnf4ref.so is not built here")
    return Reference()


@pytest.fixture(scope="session")
def package():
    return importlib.import_module("riftco-transformer_amd")


@pytest.fixture(scope="session")
def library(package):
    return package.load_library()


@pytest.fixture(scope="session")
def gpu(package, library):
    """The device plumbing module; fails (never skips) when the HIP path cannot
    run, so that a GPU run cannot pass on anything but the kernels."""
    import torch
    assert torch.cuda.is_available(), "a -m gpu test needs a visible GPU"
    assert library.is_available(), library.last_error()
    return importlib.import_module("riftco-transformer_amd.device")
