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


def test_null_operands_are_refused_before_any_device_work():
    """A null data or shape pointer with work to do is an error return, never a launch."""
    lib = _lib.load()
    sz = ctypes.c_size_t
    shape = (sz * 2)(4, 8)
    one = ctypes.c_void_p(256)  # never dereferenced on the host: every call below fails in validation
    ptrs = (ctypes.c_void_p * 2)(None, None)
    calls = [
        lambda: lib.litenn_hip_zero(0, None, 0, 16),
        lambda: lib.litenn_hip_convert(0, 0, None, 16, 5, one, None),
        lambda: lib.litenn_hip_copy_to_host(0, 0, None, 16, 0, one, None),
        lambda: lib.litenn_hip_copy_from_host(0, 0, one, 0, None, 16, None),
        lambda: lib.litenn_hip_unary(0, 0, None, 0, shape, 2, one, None),
        lambda: lib.litenn_hip_unary(0, 0, one, 0, None, 2, one, None),
        lambda: lib.litenn_hip_binary(0, 0, one, 0, shape, 2, None, 0, shape, 2, one, None),
        lambda: lib.litenn_hip_reduce(0, 0, one, 0, shape, 2, None, 1, None),
        lambda: lib.litenn_hip_concat(0, one, 0, ptrs, shape, 2, 1, 0, None),
        lambda: lib.litenn_hip_slice(0, None, 0, shape, 2, one, 0, 0, 2, None),
        lambda: lib.litenn_hip_get_rows(0, one, 0, shape, 2, one, 2, shape, 1, None, None),
        lambda: lib.litenn_hip_permute(0, one, 0, shape, 2, one, None, None),
        lambda: lib.litenn_hip_mul_mat_q(0, 9, None, 4, 256, one, 0, 1, one, None, 0, None),
        lambda: lib.litenn_hip_dequantize(0, 9, None, 4, 256, one, None),
        lambda: lib.litenn_hip_get_rows_q(0, 9, one, 4, 256, None, 1, one, None),
        lambda: lib.litenn_hip_rmsnorm(0, None, one, 1e-5, 1, 64, one, None),
        lambda: lib.litenn_hip_rope_interleaved(0, None, one, 1, 1, 64, 64, 1e4, 1.0, 0, None),
        lambda: lib.litenn_hip_kv_append(0, None, 5, 0, one, 1, 64, None),
        lambda: lib.litenn_hip_attn_decode(0, one, None, one, 5, 1, 3, 2, 2, 64, one, None),
        lambda: lib.litenn_hip_attn_rows(0, one, one, one, 5, 16, 0, 2, 2, 128, None, 0, None),
        lambda: lib.litenn_hip_silu_mul(0, one, None, one, 8, None),
        lambda: lib.litenn_hip_argmax(0, None, 1, 8, one, None),
    ]
    for i, call in enumerate(calls):
        assert call() != 0, i
        assert b"null" in lib.litenn_hip_last_error(), (i, lib.litenn_hip_last_error())
    assert lib.litenn_hip_alloc(0, 1, (1 << 63), ctypes.byref(ctypes.c_void_p())) != 0
    assert b"overflows" in lib.litenn_hip_last_error()


def test_nothing_but_the_declared_entry_points_is_exported():
    """The dynamic symbol table holds the header's functions only (linker version script)."""
    import shutil
    import subprocess
    import pytest
    nm = shutil.which("nm")
    if nm is None:
        pytest.skip("nm is not installed")
    out = subprocess.run([nm, "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.split()[-2:-1] and line.split()[-2] in "TDBR")
    assert exported == declared_symbols(), sorted(set(exported) ^ set(declared_symbols()))
