import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.pyoracle import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def reference():
    """The reference's own kernels, when oracle/_ref/libvxref.so was built."""
    from oracle.pyoracle import Reference
    if not Reference.available():
        pytest.skip("oracle/_ref/libvxref.so not built (reference tree absent at build time)")
    return Reference()


@pytest.fixture(scope="session")
def ctx():
    import torch
    import volvoxai_amd as vx
    assert torch.cuda.is_available(), "GPU tests need a device"
    c = vx.Context(0, torch.cuda.current_stream())
    yield c
    c.close()
