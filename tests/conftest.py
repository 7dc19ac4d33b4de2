import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "mojo-linuxperiments_amd"), os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    import cpu_oracle
    cpu_oracle.lib()
    return cpu_oracle


@pytest.fixture(scope="session")
def mi():
    """The HIP library through its C ABI.  Fails loudly when it is not built."""
    import mi355_int8
    return mi355_int8


@pytest.fixture(scope="session")
def dev(mi):
    d = mi.Device(arena_bytes=6 << 30)
    yield d
    d.close()
