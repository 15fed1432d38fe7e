import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU checker, registered as the host side of ``tannic_amd.ops``."""
    import support
    lib = support.oracle_library()
    import tannic_amd
    tannic_amd.ops.set_host_functions(lib.functions)
    return lib


@pytest.fixture(scope="session")
def reference():
    """The real reference CPU backend, where it could be built (oracle/_ref)."""
    import support
    lib = support.reference_library()
    if lib is None:
        pytest.skip("oracle/_ref/libtannic_ref.so is not built (needs /root/reference)")
    return lib


@pytest.fixture(scope="session")
def device(oracle):
    import tannic_amd
    return tannic_amd.Device(0)
