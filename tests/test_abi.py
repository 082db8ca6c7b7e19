"""The C-ABI library builds, loads and exports exactly what include/mlora.h declares (no compute calls)."""
import ctypes
import os
import re

import pytest

from conftest import ROOT, load_pkg


def _declared():
    text = open(os.path.join(ROOT, "include", "mlora.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mlora_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib_mod = load_pkg("_lib")
    if not os.path.exists(lib_mod.LIB_PATH):
        load_pkg("build").build()
    lib = ctypes.CDLL(lib_mod.LIB_PATH)
    names = _declared()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} declared in mlora.h but not exported"
    assert sorted(lib_mod.SIGNATURES) == names, "ctypes signature table and header disagree"
    assert lib.mlora_version() == 1


def test_argument_validation_without_gpu():
    """Shape checks happen on the host before any launch, so they can be exercised without a GPU."""
    lib = load_pkg("_lib").lib()
    assert lib.mlora_gather_mm(1, 0, 64, 1, 0, 1, 1, 1, 1.0, 4, 64, 64, 12, 2, 1, 1 << 20, None) == -2
    assert b"rank" in lib.mlora_last_error()
    assert lib.mlora_gather_mm_workspace_bytes(64, 4096, 16) == 8 * 64 * 16 * 4
    assert lib.mlora_gather_mm_workspace_bytes(32, 11008, 64) == 8 * 32 * 64 * 4
    assert lib.mlora_packed_weight_elems(40, 64) == 48 * 64
    assert lib.mlora_gemv(1, 0, 0, 1, 64, 1, 65, 64, 64, None) == -2
    assert lib.mlora_gemv(1, 0, 1, 1, 64, 1, 4, 64, 64, None) == -2          # accumulate into fp16
    assert lib.mlora_gemv(1, 1, 0, 1, 60, 1, 4, 64, 64, None) == -1          # ldx < K
    assert lib.mlora_rmsnorm(1, 0, 1, 0, 1, 1e-5, 4, 12, None) == -2
    assert lib.mlora_rmsnorm(1, 1, 1, 0, 1, 1e-5, 65, 64, None) == -2        # fragment order needs T <= 64
    assert lib.mlora_frag_activation_elems(17, 64) == 32 * 64 and lib.mlora_frag_activation_elems(33, 64) == 64 * 64
    assert lib.mlora_paged_attn_decode(1, 0, 1, 1, 1, 1, 4, 1, 1, 2, 8, 8, 96, 4, 2, None) == -2   # head_dim 96
    assert lib.mlora_paged_attn_decode(1, 0, 1, 1, 1, 1, 4, 1, 1, 2, 8, 3, 128, 4, 2, None) == -1  # Hq % Hkv


def test_ops_refuse_cpu_tensors():
    import torch
    ops = load_pkg("ops")
    x = torch.zeros(4, 64, dtype=torch.float16)
    with pytest.raises(ValueError):
        ops.rmsnorm(x, torch.ones(64, dtype=torch.float16), 1e-5)
    with pytest.raises(ValueError):
        ops.linear(x, torch.zeros(8, 64, dtype=torch.float16))
