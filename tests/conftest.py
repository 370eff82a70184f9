import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU and the built HIP kernels")


@pytest.fixture
def cpu_ops(monkeypatch):
    """Put the torch stand-ins of tests/torch_ops.py in place of the HIP
    kernels, so that the engine's bookkeeping can be tested without a GPU."""
    import torch_ops
    from litinfer_amd.kernels import ops
    for name in torch_ops.ALL:
        monkeypatch.setattr(ops, name, getattr(torch_ops, name))
    return torch_ops
