import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session", autouse=True)
def built_library():
    """The tests load the library that is built.  They compile it (hipcc
    cross-compiles without a GPU) when there is none; on a machine without a
    GPU, where sources get edited, also when a source file is newer than the
    library, so that a stale build is not what gets tested.  A GPU box runs
    the library it was sent."""
    import torch
    from habitat_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH) or (torch.cuda.device_count() == 0 and build.is_stale()):
        build.build()
    return _lib.LIB_PATH


@pytest.fixture(scope="session")
def occupancy_golden():
    """(arrays, {device name: constructor kwargs}) written by
    tests/golden/make_occupancy_golden.py from the compiled reference."""
    arrays = np.load(os.path.join(GOLDEN, "occupancy_golden.npz"))
    with open(os.path.join(GOLDEN, "occupancy_golden_devices.json")) as f:
        devices = json.load(f)
    return arrays, devices


@pytest.fixture(scope="session")
def kat():
    with open(os.path.join(GOLDEN, "kat.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def oracle_lib():
    from oracle import lib
    lib.oracle()
    return lib


def oracle_device(props):
    from oracle import lib
    return lib.make_device(**{k: v for k, v in props.items() if k != "name"})
