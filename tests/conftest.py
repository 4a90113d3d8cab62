import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for path in (ROOT, os.path.join(ROOT, "tests")):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu_ctx():
    """One context for the whole GPU session.  Creating it fails loudly when the HIP library
    is missing or no gfx950 device is visible — there is no CPU path to fall back to."""
    import karume_amd

    ctx = karume_amd.acquire_gpu(0)
    yield ctx
    ctx.destroy()
