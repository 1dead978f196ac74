import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) device; run with -m gpu")


@pytest.fixture(scope="session")
def hip_ctx():
    """One device context for the whole GPU session (raises if the HIP library is not built
    or no gfx950 device is present -- there is no fallback)."""
    from nncase_amd.runtime import Context
    ctx = Context(0)
    yield ctx
    ctx.close()
