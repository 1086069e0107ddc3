import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture
def host_device():
    """A fresh recording device seam for CPU tests of the host logic."""
    from dynaflow_amd.runtime import device as dev

    previous = dev._device
    recorder = dev.HostDevice()
    dev.set_device(recorder)
    yield recorder
    dev.set_device(previous)


def load_golden(name):
    import json

    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)
