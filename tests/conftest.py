import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def dev():
    """One Device for the whole session.  GPU tests fail (not skip) when the
    library is missing; they are skipped only where no GPU exists."""
    from vkgrad_amd.vk import Device, VkError
    try:
        d = Device()
    except VkError as e:
        if "no HIP device" in str(e):
            pytest.skip("no GPU in this machine")
        raise
    yield d
    d.destroy()
