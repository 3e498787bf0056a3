"""Shared fixtures.  GPU tests are marked `gpu`; everything else runs on a CPU-only box.

The oracle (oracle/libboat_oracle.so) and, where present, the compiled reference
(oracle/_ref/libboat_ref.so) are checkers: they are loaded here and nowhere in the product.
"""
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import oracle_lib
    return oracle_lib.load()


@pytest.fixture(scope="session")
def ref():
    """The compiled reference, or skip when it was not built (it needs the reference tree)."""
    import oracle_lib
    api = oracle_lib.load_reference()
    if api is None:
        pytest.skip("oracle/_ref/libboat_ref.so not built (reference tree absent at build time)")
    return api


@pytest.fixture(scope="session")
def hip():
    from boat_amd import hip as h
    h.check(h.bh_init(), "bh_init")
    return h


@pytest.fixture(scope="session")
def boat(hip):
    from boat_amd.capi import default_api
    return default_api()


@pytest.fixture
def rng(request):
    import zlib
    seed = zlib.crc32(request.node.nodeid.encode()) % (2**31)     # the same data in every run (str hashes change per process)
    return np.random.default_rng(seed)
