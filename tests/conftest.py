import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for path in (ROOT, os.path.join(ROOT, "tests")):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def device():
    """One device for the whole GPU session; a missing HIP library or GPU is a failure, not a skip."""
    import neura_amd

    held = neura_amd.Device(0)
    yield held
    held.close()
