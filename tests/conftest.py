import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def shim_built():
    """The C-ABI library must already be built (``__graft_entry__.build()``)."""
    from loopfuse_amd import runtime

    if not os.path.exists(runtime.SHIM_PATH):
        import __graft_entry__

        __graft_entry__.build_shim()
    return runtime.lib()
