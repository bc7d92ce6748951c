import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as O

    O.lib()
    return O


@pytest.fixture(scope="session")
def hip():
    """The C ABI on a box with a GPU; fails (not skips) when the library or the device is missing."""
    from openvino_contrib_amd import capi

    capi.lib()
    assert capi.device_count() > 0, "no HIP device: GPU tests must run on the GPU box"
    capi.check(capi.lib().hipattn_set_device(0))
    return capi


@pytest.fixture
def schedule_options(hip):
    """Sets process-wide schedule options of the library for one test and restores the defaults after it."""
    touched = []

    def apply(options):
        for name, value in options.items():
            hip.set_option(name, value)
            touched.append(name)

    yield apply
    for name in touched:
        hip.set_option(name, -1)
