import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import knet_oracle
    knet_oracle.lib()  # builds oracle/libknet_oracle.so with gcc if it is missing
    return knet_oracle


@pytest.fixture(scope="session")
def knet():
    """The host-side mirror of the reference interface, backed by libknet8.so (HIP)."""
    import __graft_entry__ as ge
    if not os.path.exists(os.path.join(ROOT, "knet.jl_amd", "lib", "libknet8.so")):
        ge.build()  # nothing built yet (fresh checkout): cross-compile once; otherwise load what is there
    return ge.load_package()
