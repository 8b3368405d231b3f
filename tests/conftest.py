import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import uk_oracle
    return uk_oracle.get("oracle")


@pytest.fixture(scope="session")
def reference():
    """The compiled reference ukernels (oracle/_ref); tests that need it are
    skipped where it was not built."""
    from oracle import uk_oracle
    if not uk_oracle.Checker.reference_available():
        pytest.skip("oracle/_ref/libiree_uk_ref.so not built")
    return uk_oracle.get("reference")


@pytest.fixture(scope="session")
def lib():
    """The product library. Built beforehand by `python -m iree_amd.build`;
    only if nothing is built is it compiled here."""
    from iree_amd import ukernel
    if not os.path.exists(ukernel.LIB_PATH):
        from iree_amd import build
        build.build()
    L = ukernel.load()
    L.raise_on_violation(True)
    return L


@pytest.fixture(scope="session")
def gpu(lib):
    """(lib, torch) with the GPU initialised; GPU tests fail loudly without one."""
    import torch
    assert torch.cuda.is_available(), "GPU test selected but no GPU is visible"
    assert lib.device_count() >= 1
    torch.cuda.init()
    lib.set_stream(None)
    return lib, torch
