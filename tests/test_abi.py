"""The C-ABI library: loads without a GPU, exports what include/forge_hip.h declares, and
rejects bad arguments before touching the device."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]


def _declared():
    text = (ROOT / "include" / "forge_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(forge_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    from forge.backend.hip import load_library, EXPORTED_SYMBOLS
    lib = load_library()
    names = _declared()
    assert len(names) >= 16
    for n in names:
        assert hasattr(lib, n), f"{n} declared in forge_hip.h but not exported"
    assert sorted(EXPORTED_SYMBOLS) == names
    assert lib.forge_hip_abi_version() == 1


def test_invalid_arguments_are_rejected_without_a_launch():
    from forge.backend.hip import load_library
    lib = load_library()
    rc = lib.forge_mse_scale_groups_packed(None, None, None, None, 4, 48, 3, 2.4, 4, 1, None)
    assert rc == 1 and b"group_size=48" in lib.forge_last_error()
    rc = lib.forge_gptq_solver(None, None, None, None, 4, 128, 64, None, None, None)
    assert rc == 1 and b"null pointer" in lib.forge_last_error()
    rc = lib.forge_quant_grid(None, 7, 1, 0, 4, 128, 128, 128, 4, 1, 0, None, 0, 2.4, None, None, None)
    assert rc == 1 and b"w_dtype" in lib.forge_last_error()
    assert lib.forge_build_group_meta_packed(None, 0, 128, 4, 1, None, None, None) == 0   # empty: no-op
    # inverse diagonal blocks (fp32) + the 16-bit pieces of two 128-column panels (6 bytes per
    # element each) + one fp32 scale per column
    assert lib.forge_chol_workspace_bytes(2, 256) == 2 * 2 * 128 * 128 * 4 + 2 * 2 * 256 * 128 * 6 + 2 * 256 * 4


def test_options_are_settings_of_the_library_not_of_the_environment(monkeypatch):
    from forge.backend.hip import load_library
    lib = load_library()
    assert lib.forge_get_option(b"sweep_update_products") == 0
    assert lib.forge_get_option(b"sweep_schedule") == 0
    monkeypatch.setenv("FORGE_SWEEP_SCHEDULE", "right")          # read at load time only
    assert lib.forge_get_option(b"sweep_schedule") == 0
    assert lib.forge_set_option(b"sweep_schedule", 2) == 0 and lib.forge_get_option(b"sweep_schedule") == 2
    assert lib.forge_set_option(b"sweep_schedule", 0) == 0
    assert lib.forge_set_option(b"sweep_update_products", 5) == 1
    assert b"not allowed" in lib.forge_last_error()
    assert lib.forge_set_option(b"no_such_option", 1) == 1 and lib.forge_get_option(b"no_such_option") == -1


@pytest.mark.skipif(torch.cuda.is_available(), reason="CPU-only behaviour")
def test_no_cpu_fallback():
    from forge.backend.hip import kernels
    with pytest.raises(RuntimeError, match="unavailable"):
        kernels.gptq_solver
    from forge.gptq import GPTQ
    with pytest.raises(RuntimeError, match="GPU only"):
        GPTQ(torch.nn.Linear(8, 8), device="cpu")
