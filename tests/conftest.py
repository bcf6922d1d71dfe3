import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests"), os.path.join(ROOT, "go-metal_amd")):   # workloads.py lives in the package
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_sessionstart(session):
    """Loads what is built; builds only when nothing is (a fresh checkout): the library and the
    CPU checker are git-ignored artefacts."""
    lib = os.path.join(ROOT, "go-metal_amd", "libgometal_hip.so")
    oracle_lib = os.path.join(ROOT, "oracle", "liboracle.so")
    client = os.path.join(ROOT, "tests", "c_client", "abi_client.bin")
    if not os.path.exists(lib) or not os.path.exists(oracle_lib) or not os.path.exists(client):
        import __graft_entry__
        __graft_entry__.build()
