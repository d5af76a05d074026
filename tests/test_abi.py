"""CPU checks of the boundary: the shared library loads without a GPU, exports every symbol that
include/rwkv_hip.h declares, and argument errors come back as error codes (never a crash or exit)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "rwkv_hip.h")).read()
    return sorted(set(re.findall(r"\b(rwkv_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from rwkv_lightning_cuda_amd import hip
    lib = hip.load()
    names = declared_symbols()
    assert len(names) >= 55
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(hip.EXPORTS) == names


def test_errors_are_codes_not_crashes():
    from rwkv_lightning_cuda_amd import hip
    lib = hip.load()
    assert hip.device_count() >= 0
    # shape checks run on the host before anything touches a device
    rc = lib.rwkv_hip_wkv7(None, 1, 1, 100, 1, 0, 0, None, None, None, None, None, None, None, None)
    assert rc == -1 and b"H*64" in lib.rwkv_hip_last_error()
    m = ctypes.c_void_p(0)
    assert lib.rwkv_hip_model_create(ctypes.byref(m), 1, 100, 1, 64, 64, 8, 8, 8, 8) == -1
    assert b"C must equal H*N" in lib.rwkv_hip_last_error()
    assert lib.rwkv_hip_model_create(ctypes.byref(m), 1, 64, 1, 64, 64, 8, 8, 8, 1024) == -1
    assert lib.rwkv_hip_model_create(ctypes.byref(m), 2, 64, 1, 64, 64, 8, 8, 8, 8) == 0
    assert lib.rwkv_hip_model_set_tensor(m, 5, 10, ctypes.c_void_p(16)) == -1      # layer out of range
    assert lib.rwkv_hip_model_set_matrix(m, 0, 0, 1, ctypes.c_void_p(16), None, None) == -1   # W8 without scale
    assert lib.rwkv_hip_model_set_matrix(m, 0, 0, 2, ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16)) == -1  # W4, K=64
    n = ctypes.c_uint64(0)
    assert lib.rwkv_hip_model_weight_bytes(m, ctypes.byref(n)) == 0 and n.value > 0
    assert lib.rwkv_hip_model_destroy(m) == 0
    assert lib.rwkv_hip_sample(None, 1, 6, None, None, None, None, ctypes.c_double(0), ctypes.c_double(0),
                               ctypes.c_double(1), ctypes.c_double(1), 0, ctypes.c_double(1), ctypes.c_uint64(0),
                               ctypes.c_uint64(0)) == -1
    assert b"multiple of 4" in lib.rwkv_hip_last_error()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from rwkv_lightning_cuda_amd import hip
    monkeypatch.setattr(hip, "_lib", None)
    monkeypatch.setattr(hip, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(hip.RwkvHipError, match="no CPU fallback"):
        hip.load()
