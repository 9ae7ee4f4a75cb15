import sys
from pathlib import Path

import pytest
# Some GPU tests use torch as the owner of device memory and streams.  torch ships a HIP runtime of its own under the same
# soname as the system's; whichever of torch and libjitnn_hip.so is loaded first decides which copy the process uses,
# and only with torch first do both end up on one runtime (the other order gives two, and the second to touch the GPU
# finds "no ROCm-capable device").  So torch is loaded here, before any test module can load the library.
import torch  # noqa: F401

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def goldens():
    from helpers import load_goldens
    return load_goldens()


@pytest.fixture(scope="session")
def gguf_fixture():
    from helpers import fixture
    return fixture()
