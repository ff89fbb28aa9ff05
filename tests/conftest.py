import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Without a GPU the host runtime hands out addresses only (graph construction and
# lowering still work); with a GPU this variable is ignored.
os.environ.setdefault("MIRAGE_HOST_ONLY", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def _have_gpu() -> bool:
    return os.path.exists("/dev/kfd") and os.path.exists("/dev/dri")


@pytest.fixture(scope="session")
def rt():
    """The host runtime with a GPU attached; GPU tests fail loudly without one."""
    from attention_superoptimizer_amd import graph as G
    assert _have_gpu(), "no GPU device nodes: GPU tests need an MI355X"
    assert G.device_ready(), "runtime came up in host-only mode on a GPU box"
    G.set_smem_budget(1 << 20)
    return G


@pytest.fixture(scope="session")
def abi(rt):
    from attention_superoptimizer_amd import _native as N
    return N.backend()
