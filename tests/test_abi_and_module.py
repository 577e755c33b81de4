"""CPU-side checks of the drop-in boundary: the C ABI library loads and exports exactly what
include/f3s_amd.h declares, and the `F3S` operator module has the reference's six entry points
with the reference's error behaviour for non-device tensors (src/F3S.cpp:12-18,156-161,298-305)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "f3s_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(f3s_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from fused3s_amd import capi
    lib = ctypes.CDLL(capi.LIB_PATH)
    names = declared_symbols()
    assert set(names) == set(capi.EXPORTS)
    for n in names:
        assert getattr(lib, n) is not None
    lib.f3s_abi_version.restype = ctypes.c_int
    assert lib.f3s_abi_version() == 2
    lib.f3s_last_error.restype = ctypes.c_char_p
    assert isinstance(lib.f3s_last_error(), bytes)
    lib.f3s_preprocess_workspace_bytes.restype = ctypes.c_size_t
    lib.f3s_preprocess_workspace_bytes.argtypes = [ctypes.c_int, ctypes.c_int]
    assert lib.f3s_preprocess_workspace_bytes(1000, 5000) >= 256 + 3 * 63 * 4


def test_argument_errors_are_statuses_not_exits():
    """Host-side argument checks run before any GPU work, so they are testable without a GPU."""
    from fused3s_amd import capi
    L = capi.lib()
    rc = L.f3s_attention_fwd(None, None, None, None, -1, 0, 64, 0, None, None, None, 1.0, 1, None,
                             None, None, 0, 0, None)
    assert rc != 0 and b"negative" in L.f3s_last_error()
    rc = L.f3s_attention_fwd(None, None, None, None, 5, 0, 64, 0, None, None, None, 1.0, 1, None,
                             None, None, 0, 0, None)
    assert rc != 0 and b"null" in L.f3s_last_error()
    n = ctypes.c_int64(0)
    rc = L.f3s_preprocess_count(None, None, 5, 0, 16, 16, None, None, None, None, None, None, 0,
                                ctypes.byref(n), None)
    assert rc != 0


def test_module_surface_matches_reference():
    from fused3s_amd import F3S
    for name in ["preprocess_gpu", "f3s_1tb1tcb", "f3s_1tb1rw", "f3s_1tb1rw_scheduled",
                 "f3s_1tb1rw_scheduled_permuteV", "f3s_1tb1rw_scheduled_permuteV_scaleQK"]:
        assert callable(getattr(F3S, name))


def test_cpu_tensors_raise_runtime_error():
    from fused3s_amd import F3S
    i32 = torch.zeros(2, dtype=torch.int32)
    h = torch.zeros(1, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        F3S.f3s_1tb1rw(i32, torch.zeros(16, dtype=torch.int32), torch.zeros(4, dtype=torch.int64),
                       1, h, h, h, 8, True, False)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        F3S.f3s_1tb1tcb(i32, torch.zeros(8, dtype=torch.int32), torch.zeros(2, dtype=torch.int64),
                        1, h, h, h, True, False)
    with pytest.raises(RuntimeError):
        F3S.preprocess_gpu(torch.zeros(1, dtype=torch.int32), i32, 1, 16, 16,
                           torch.zeros(1, dtype=torch.int32), torch.zeros(1, dtype=torch.int32),
                           torch.zeros(1, dtype=torch.int32))


def test_product_does_not_import_the_oracle():
    """The shipped package must never route through the CPU oracle."""
    pkg = os.path.join(ROOT, "fused3s_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "f3s_oracle" not in text, f
