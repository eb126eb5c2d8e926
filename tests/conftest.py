import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_addoption(parser):
    parser.addoption("--host-sanitizers", action="store_true", default=False,
                     help="also run tests/host_sanitizers.py (ASan + UBSan builds of the host C++ "
                          "layer and the oracle under the CPU tests; about two minutes)")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


def pytest_collection_modifyitems(config, items):
    # GPU tests are only meaningful with a device; without one they are skipped, never faked.
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as orc
    orc.lib()
    return orc


def announce(msg):
    """Name the case on stdout before a GPU step so a lost box still tells which case ran."""
    print("[gpu-case] " + msg, flush=True)
