"""Shared pytest configuration.

``gpu``-marked tests need a real MI355X and the built HIP library; everything
else runs on the CPU (oracle against golden vectors, host logic, symbol
export checks).
"""

import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # GPU tests load the library that is built in the tree; it is compiled here only if
    # there is none (the package itself never builds: a missing library is an error there)
    if "not gpu" in (config.getoption("markexpr", "") or ""):
        return
    if any("gpu" in item.keywords for item in items):
        import __graft_entry__
        __graft_entry__.ensure_built()
