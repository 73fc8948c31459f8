import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _ensure_built():
    need = ["spcomm3d_amd/lib/libspcomm3d_hip.so", "spcomm3d_amd/gen/libspc3d_gen.so",
            "oracle/liboracle.so"]
    if not all(os.path.exists(os.path.join(ROOT, p)) for p in need):
        import __graft_entry__

        __graft_entry__.build()


_ensure_built()


@pytest.fixture(scope="session")
def ctx():
    """One device context for the whole GPU session; fails loudly without a GPU."""
    from spcomm3d_amd import device

    c = device.Context(0)
    yield c
    c.close()
