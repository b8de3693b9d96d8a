"""The C++ host side (include/LiteNN/Device/HIP.h: DeviceTraits<HIP> with the reference's member
names over the C ABI), exercised by tests/cpp/device_traits_test.cpp, which mirrors the reference's
device tests (tests/CUDADeviceTest.cpp:69-125) and its Q4_0 payload fixture
(tests/GGUFImporterTest.cpp:173-178).  The binary is built by `python -m litenn_amd.build`."""
import os
import subprocess

import pytest

from litenn_amd import build as hip_build


def run_binary():
    assert os.path.exists(hip_build.CPP_TEST_BIN), "run `python -m litenn_amd.build` (or __graft_entry__.build())"
    return subprocess.run([hip_build.CPP_TEST_BIN], capture_output=True, text=True, timeout=120)


def test_cpp_header_compiles_and_device_free_checks_pass():
    """No GPU needed: the error path and the no-device behaviour of the traits."""
    p = run_binary()
    assert p.returncode == 0, p.stdout + p.stderr
    assert "FAIL" not in p.stdout
    assert "unsupported block format throws" in p.stdout


@pytest.mark.gpu
def test_cpp_device_traits_on_the_gpu():
    p = run_binary()
    assert p.returncode == 0, p.stdout + p.stderr
    assert "all checks passed" in p.stdout, p.stdout
    for name in ("MatMul reference vector", "Q4_0 fixture block . x", "Q4_0 fixture block dequantised",
                 "RMSNorm closed form", "Reduce Sum"):
        assert f"ok   {name}" in p.stdout, p.stdout


def test_fetch_patterns_stay_inside_their_tensors():
    """tests/cpp/fetch_bounds_test.cpp (CPU only): the address arithmetic the kernels call
    (litenn_amd/csrc/fetch_model.hpp) walked for every thread of a launch -- matrix-core GEMM weight
    pieces for every format, tile and misalignment including page-exact tensors, streaming GEMV rows
    with the lane-0 fill-in, activation loads, attention key tiles -- and the GEMM's arithmetic as
    it was before its over-fetch was fixed, which must be caught."""
    assert os.path.exists(hip_build.FETCH_TEST_BIN), "run `python -m litenn_amd.build` (or __graft_entry__.build())"
    p = subprocess.run([hip_build.FETCH_TEST_BIN], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stdout[-3000:] + p.stderr
    assert "fetch bounds ok" in p.stdout and "FAIL" not in p.stdout
    assert "pieces behind the tensor before the fix, 0 now" in p.stdout
