import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_addoption(parser):
    parser.addoption("--emulate", action="store_true",
                     help="run the tests marked gpu without a GPU, on the host build of the kernel sources "
                          "(tests/emu_lib.py); --emulate-order and --emulate-eager choose the lane order and when "
                          "LDS-direct loads land")
    parser.addoption("--ubsan", action="store_true",
                     help="also run test_emulated_kernels.py's sanitizer pass (builds the host model with the undefined-"
                          "behaviour sanitizer: minutes)")
    parser.addoption("--mutants", action="store_true",
                     help="run test_host_model_mutants.py (a build of the host model per seeded mistake: minutes)")
    parser.addoption("--emulate-order", type=int, default=0)
    parser.addoption("--emulate-eager", action="store_true")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "needs_device: uses streams, graphs or timing that only a real device has")
    if config.getoption("--emulate"):
        import emu_lib
        emu_lib.install()
        emu_lib.configure(order=config.getoption("--emulate-order"), lazy_loads=not config.getoption("--emulate-eager"))


def _gpu_available():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if config.getoption("--emulate"):
        skip = pytest.mark.skip(reason="needs a real device")
        for item in items:
            if "needs_device" in item.keywords:
                item.add_marker(skip)
        return
    if _gpu_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_sessionfinish(session, exitstatus):
    """Host-model runs leave what the model executed (per kind of wave-wide operation: all, and those that ran with
    part of their wave because the wave had diverged) beside the build, one file per process."""
    if not session.config.getoption("--emulate"):
        return
    import json
    import emu_lib
    path = os.path.join(emu_lib.BUILD, "counts_%d.json" % os.getpid())
    with open(path, "w") as f:
        json.dump(emu_lib.counts(), f)
