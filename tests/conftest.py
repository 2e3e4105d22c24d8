import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (ROOT, ROOT / "sonic-moe_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture
def tuning():
    """Set kernel-selection knobs of the HIP library for one test: tuning(name, value); defaults are restored after."""
    from sonicmoe import _lib

    touched = []

    def set_knob(name, value):
        _lib.set_tuning(name, value)
        touched.append(name)

    yield set_knob
    for name in touched:
        _lib.set_tuning(name, -1)
