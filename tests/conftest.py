"""Shared test plumbing: marker registration, package import, oracle import, GPU library handle."""

import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    """The product package (its directory name has a hyphen, so it is imported through the entry module)."""
    import __graft_entry__ as entry

    return entry.import_package()


@pytest.fixture(scope="session")
def oracle():
    from oracle import raven_oracle

    return raven_oracle


@pytest.fixture(scope="session")
def lib(pkg):
    """The loaded C-ABI library; GPU tests fail (not skip) when it is missing."""
    return pkg.hip.load()
