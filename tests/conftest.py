import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for sub in ("torch-ash_amd", "oracle", ""):
    path = os.path.join(ROOT, sub) if sub else ROOT
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle as a backend object (HashMap class + query functions)."""
    import ash_oracle

    return ash_oracle.OracleBackend()


@pytest.fixture()
def cpu_ash(oracle, monkeypatch):
    """The package's Python layer wired to the CPU oracle, so host-side logic
    (engines, modules, neighbour tables, autograd wiring) runs without a GPU.
    Only tests do this; the package itself has no CPU path."""
    import ash
    import ash.core
    import ash.grid
    import ash.grid_query

    for mod in (ash.core, ash.grid, ash.grid_query):
        monkeypatch.setattr(mod, "backend", oracle)
    return ash


@pytest.fixture(scope="session")
def gpu_ash():
    """The package on the real device; fails loudly if the HIP library or the
    device is missing."""
    import torch

    assert torch.cuda.is_available(), "gpu tests need a HIP device"
    import ash
    from ash.common import _Backend

    assert isinstance(ash.core.backend, _Backend), "libash_hip.so is not loaded"
    return ash
