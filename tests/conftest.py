import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session", autouse=True)
def _native_libraries():
    """Load what is built; compile only if nothing is (a fresh checkout has no .so files)."""
    from xccl_amd import build
    if not build.built():
        build.build(force=False)


def _have_gpu() -> bool:
    try:
        from xccl_amd import hip
        return hip.device_count() > 0
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import pyoracle
    pyoracle.lib()
    return pyoracle


@pytest.fixture(scope="session")
def rocm():
    """The dispatcher with the ROCm component loaded, on device 0."""
    from xccl_amd import hip, mc
    from xccl_amd.types import MemType, Status
    assert hip.device_count() > 0
    hip.set_device(0)
    assert mc.xccl_mem_component_init() == Status.OK
    assert bool(mc.dispatch_lib().xccl_mem_component_get(int(MemType.ROCM))), \
        "xccl_rocm_mem_component.so was not loaded by the dispatcher"
    return mc
