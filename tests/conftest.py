import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT))                       # oracle/
sys.path.insert(0, str(ROOT / "4bit-forge_amd"))    # forge/


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP kernels through the C ABI)")


@pytest.fixture(scope="session")
def hip():
    """The operator table; GPU tests fail loudly if the HIP library did not load."""
    import torch
    from forge.backend.hip import kernels
    assert torch.cuda.is_available(), "GPU test collected without a GPU"
    kernels.build_group_meta_packed  # raises RuntimeError if libforge_hip.so is missing
    return kernels
