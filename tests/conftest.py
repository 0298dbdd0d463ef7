import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _build_missing():
    """Tests load what is built; they build only what is absent or was built from other sources than
    the ones on disk (CPU-side libraries and, by cross-compilation, the HIP library)."""
    from fasterllama_amd import build
    for name in ("oracle", "synth", "hip"):
        if build.is_stale(name):
            build.TARGETS[name]()


@pytest.fixture(scope="session", autouse=True)
def native_libs():
    _build_missing()
    yield


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("this test is marked gpu and needs a GPU; run CPU suites with -m 'not gpu'")
    return torch.device("cuda:0")
