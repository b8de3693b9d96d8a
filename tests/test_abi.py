"""The C-ABI library loads and exports every symbol the public header declares (no GPU, no
compute calls)."""
import ctypes
import os
import re

from litenn_amd import _lib


def declared_symbols():
    text = open(_lib.HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(litenn_(?:hip|gguf)_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built_in_tree():
    assert os.path.exists(_lib.LIB_PATH), "run `python -m litenn_amd.build` (or __graft_entry__.build())"


def test_every_declared_symbol_is_exported():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 30
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_python_binding_covers_the_header():
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_device_count_never_fails_and_errors_are_reported_without_a_device():
    lib = _lib.load()
    count = lib.litenn_hip_device_count()
    assert count >= 0
    if count == 0:
        out = ctypes.c_void_p()
        assert lib.litenn_hip_alloc(0, 0, 16, ctypes.byref(out)) != 0
        assert b"HIP allocate failed" in lib.litenn_hip_last_error()
    # argument validation happens before any device work
    assert lib.litenn_hip_mul_mat_q(0, 9, None, 4, 100, None, 0, 1, None, None, 0, None) != 0
    assert b"block size" in lib.litenn_hip_last_error()
    assert lib.litenn_hip_mul_mat_q(0, 6, None, 4, 32, None, 0, 1, None, None, 0, None) != 0  # Q8_1: no dequantizer
    assert b"unsupported block format" in lib.litenn_hip_last_error()
