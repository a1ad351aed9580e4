import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (built on demand with g++)."""
    from oracle import cn_oracle

    return cn_oracle.Oracle()


@pytest.fixture(scope="session")
def dev():
    """Device helper bound to libcnhip; GPU tests only."""
    from tests.helpers import Device

    return Device()


@pytest.fixture(scope="session")
def cpu_cg_system():
    """The dense CG configuration on the host (n = 16384, oracle generator, seed 2): matrix tiles
    and right-hand side, built once per session (2 GiB)."""
    import bench

    return bench.cpu_cg_setup(16384)
