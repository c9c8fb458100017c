"""The C-ABI library loads, exports every symbol include/dmoe.h declares, and its
host-side argument checks answer without a GPU (no compute call is made)."""
import ctypes
import os
import re

import pytest

from disagmoe_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dmoe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dmoe_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 15
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in dmoe.h but not exported"
    assert sorted(_lib.SIGNATURES) == declared, "ctypes table and header disagree"
    assert _lib.version().startswith("dmoe-hip gfx950")


def test_signatures_have_no_torch_types():
    text = open(os.path.join(ROOT, "include", "dmoe.h")).read()
    code = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    assert "torch" not in code and "at::" not in code and "c10" not in code and "Tensor" not in code


def test_host_side_argument_errors():
    lib = _lib.load()
    need = ctypes.c_size_t(123)
    assert lib.dmoe_route_scratch_bytes(512, 8, ctypes.byref(need)) == 0 and need.value == 0
    assert lib.dmoe_route_scratch_bytes(49152, 64, ctypes.byref(need)) == 0 and need.value == (96 + 1) * 64 * 4
    assert lib.dmoe_route_scratch_bytes(10, 0, ctypes.byref(need)) == -2
    assert b"E=0" in lib.dmoe_last_error()
    assert lib.dmoe_gmm_workspace_bytes(8, ctypes.byref(need)) == 0 and need.value > 0
    # row length that is not a multiple of 16 bytes
    assert lib.dmoe_permute(None, None, None, 8, 4, 4, 7, 0, None, None) == -2
    # R not a multiple of T
    assert lib.dmoe_permute(None, None, None, 8, 4, 6, 8, 0, None, None) == -2
    # bad dtype / bad mapping type / null pointers
    assert lib.dmoe_permute(None, None, None, 8, 4, 4, 8, 9, None, None) == -3
    assert lib.dmoe_permute(None, None, None, 8, 4, 4, 8, 0, None, None) == -1
    assert lib.dmoe_combine(None, None, 8, None, None, 4, 0, 8, 0, 0, None) == -1
    assert lib.dmoe_gmm(None, None, None, None, 16, 8, 60, 64, 0, 0, None, None, 0, None, None) == -2      # K % 8
    assert lib.dmoe_gmm(None, None, None, None, 16, 8, 64, 64, 0, 1, None, None, 0, None, None) == -3      # fp16 not supported
    assert lib.dmoe_gmm_fp8(None, None, None, None, None, None, 16, 8, 72, 64, None, None, 0, None, None) == -2  # K % 16
    header = open(os.path.join(ROOT, "include", "dmoe.h")).read()
    assert f"#define DMOE_GMM_STATE_BYTES {_lib.GMM_STATE_BYTES}" in header
    assert "dmoe_gmm_tune" not in header and hasattr(lib, "dmoe_gmm_tune")      # a test hook, not public ABI
    assert lib.dmoe_gmm_tune(9) == -1 and lib.dmoe_gmm_tune(4) == 0 and lib.dmoe_gmm_tune(0) == 0
    with pytest.raises(_lib.DmoeError):
        _lib.call("dmoe_gmm_tune", -1)
    # empty problems succeed without touching the device
    assert lib.dmoe_permute(None, None, None, 8, 0, 0, 8, 0, None, None) == 0
    assert lib.dmoe_combine(None, None, 8, None, None, 0, 2, 8, 0, 0, None) == 0
