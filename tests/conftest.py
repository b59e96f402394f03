import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _gpu_present() -> bool:
    return os.path.exists("/dev/kfd") and os.access("/dev/kfd", os.R_OK | os.W_OK)


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU device in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


class _DeviceBufferLedger:
    """Every device buffer a test takes through the backend's malloc / to_device, until it is freed."""

    def __init__(self, be):
        self.live = set()
        malloc, free = be.malloc, be.free

        def tracked_malloc(nbytes):
            p = malloc(nbytes)
            if p:
                self.live.add(p)
            return p

        def tracked_free(dptr):
            self.live.discard(dptr)
            free(dptr)

        be.malloc, be.free = tracked_malloc, tracked_free   # to_device allocates through self.malloc


@pytest.fixture(scope="module")
def be():
    import larql_amd
    b = larql_amd.HipBackend()
    b._ledger = _DeviceBufferLedger(b)
    yield b
    b.close()


@pytest.fixture(scope="module")
def fmt():
    import larql_amd
    return larql_amd


@pytest.fixture(autouse=True)
def _free_device_buffers_of_the_test(request):
    """A GPU test's device buffers are returned when it ends, whether or not it freed them itself."""
    if "be" not in request.fixturenames:
        yield
        return
    b = request.getfixturevalue("be")
    before = set(b._ledger.live)
    yield
    b.synchronize()
    for p in list(b._ledger.live - before):
        b.free(p)
