import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _gpu_present():
    return os.path.exists("/dev/kfd")


if _gpu_present():
    # PyTorch-ROCm wheels bundle their own HIP runtime under an unversioned file
    # name.  Loaded first, it is shared by libnbhip.so (same SONAME); loaded second,
    # the process ends up with two HIP runtimes and torch no longer sees the GPU.
    # The interop test needs both, so torch goes first.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU in this machine")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def fake_gpu(monkeypatch):
    """The driver layer bound to tests/fakelib.FakeLib: device memory lives in
    host RAM, no kernels exist.  Yields the FakeLib for inspection."""
    from tests.fakelib import FakeLib
    from numba_cuda_amd.cudadrv import devices, driver as drv

    lib = FakeLib()
    d = drv.driver
    saved = dict(d.__dict__)
    for name in [k for k in d.__dict__ if k.startswith("nbh_")]:
        del d.__dict__[name]                      # drop cached checked wrappers
    d.lib, d.is_initialized, d.initialization_error, d.pid = lib, True, None, os.getpid()
    d._devices = {}                               # a table of its own for the fake devices
    devices._runtime._tls.__dict__.clear()
    devices.gpus._entries = None                  # the device list is asked for again, from the fake library
    drv._ActiveContext._tls.__dict__.clear()
    monkeypatch.setattr(drv, "_memory_manager", None)
    try:
        yield lib
    finally:
        import gc
        gc.collect()
        d.__dict__.clear()
        d.__dict__.update(saved)
        for name in [k for k in d.__dict__ if k.startswith("nbh_")]:
            del d.__dict__[name]
        devices._runtime._tls.__dict__.clear()
        devices.gpus._entries = None
        drv._ActiveContext._tls.__dict__.clear()
